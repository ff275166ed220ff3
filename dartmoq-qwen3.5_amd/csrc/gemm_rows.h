// Codebook-dequant GEMM for big batches of fp16 layers: a persistent kernel over stretches of up
// to 128 activation rows (gfx950 MFMA).
//
//   out[r, n] = sum_g sum_{k<128} a[r, g, k] * fp16(LUT[idx[g, n, k]] * norm[g, n])
//
// Same arithmetic, element for element, as the 32- and 64-row instances of dmq_gemm_gf_kernel (the
// norm is multiplied into the fp16 weight operand, the MFMAs of a (row, feature) run in the same
// order over the same K slices), so a row's bits do not depend on which kernel or tile size served
// it.  What differs is the shape of the work and its schedule:
//
//   * The table look-up that dequantizes a packed byte is the expensive part of these GEMMs, and
//     its cost per weight is the same whatever the number of activation rows.  A work item is
//     therefore a stretch of up to 128 rows of one expert: every wave dequantizes its 64 weight
//     rows of a group once into registers and contracts them against up to eight 16-row tiles
//     (TT = 8: one look-up feeds eight MFMAs; 33..64 rows run TT = 4, up to 32 rows TT = 2).
//   * One workgroup per CU, one wave per SIMD (the accumulators of 128 rows x 64 weight rows take
//     128 registers), launched once per CU and persistent: the units (work item x run of feature
//     blocks) are handed out from per-XCD queues in order of decreasing cost (TT = 8 units first),
//     so the short units of the ragged ends fill the gaps the long ones leave.
//   * A wave with the SIMD to itself hides no latency by occupancy, so everything is software
//     pipelined: packed weights and norms travel three groups ahead in a register ring, the
//     activation tile of a group goes from memory straight into one of three LDS buffers two
//     groups ahead (global_load_lds_dwordx4: no registers, no LDS store instructions, and nothing
//     waits for it until the barrier in front of the group that reads it), and inside a group the
//     scaled operands and look-ups of the following MFMA steps and the activation operands of the
//     following micro-steps (MFMA step s, row tile t) are produced between the MFMAs.
//   * The pipeline does not drain between units: while a unit runs, the workgroup draws the next
//     one from the queue (one atomic), reads its record and row indices, and directs the loads of
//     its last three groups at the next unit's first three.  Only a change of tile class or pool
//     starts from an empty pipeline.
#pragma once
#include "gemm_gf.h"

#define DMQ_ROWS_NBUF 3
#define DMQ_ROWS_STAGE_BYTES (DMQ_ROWS_NBUF * DMQ_ROWS_TILE * 256)
#define DMQ_ROWS_ORDER_OFF (DMQ_LUT_BYTES + DMQ_ROWS_STAGE_BYTES)
#define DMQ_ROWS_MAIL_OFF (DMQ_ROWS_ORDER_OFF + DMQ_ROWS_MAX_ITEMS * 2)
#define DMQ_ROWS_LDS (DMQ_ROWS_MAIL_OFF + 256)
// scheduling state is equal in all lanes; saying so keeps it (and every address built from it) in
// scalar registers and its branches scalar
#define DMQ_UNI(x) __builtin_amdgcn_readfirstlane((int)(x))

// One unit of work: a stretch of rows of one expert times a run of nbl feature blocks.
struct RowsUnit {
  int valid;
  int cls;                                // 0: up to 128 rows (TT = 8), 1: up to 64 (TT = 4), 2: up to 32 (TT = 2)
  int pool;
  int kb0;                                // first feature block of the run
  int r_first, r_end;                     // logical rows [r_first, r_end) (r_end: end of the expert's rows)
  int slice_start;                        // weight rows (gate_up) or groups (down) of the expert's slice
  int post_slice;                         // first down group of the expert (fused rotation)
  // the same unit with every field in a scalar register (the fields are equal in all lanes)
  __device__ __forceinline__ RowsUnit uniform() const {
    RowsUnit u;
    u.valid = __builtin_amdgcn_readfirstlane(valid); u.cls = __builtin_amdgcn_readfirstlane(cls);
    u.pool = __builtin_amdgcn_readfirstlane(pool); u.kb0 = __builtin_amdgcn_readfirstlane(kb0);
    u.r_first = __builtin_amdgcn_readfirstlane(r_first); u.r_end = __builtin_amdgcn_readfirstlane(r_end);
    u.slice_start = __builtin_amdgcn_readfirstlane(slice_start);
    u.post_slice = __builtin_amdgcn_readfirstlane(post_slice);
    return u;
  }
};

// Scheduling state of a workgroup (uniform over its threads).
struct RowsSched {
  int* queue;                             // DMQ_ROWS_QUEUE_WORDS device words
  const int* items;
  const uint16_t* order;                  // LDS: work items by class
  int* mail;                              // LDS
  int n;                                  // ordered items
  int nbr, nbl;                           // runs per item, blocks per run
  int wgs;                                // workgroups per XCD
  int xcd;                                // this workgroup's XCD
  int victim;                             // queues tried so far (0: own)
  int slice_is_groups;

  __device__ __forceinline__ int queue_of(int v) const { return (xcd + v) & (DMQ_XCDS - 1); }
  // queue position -> sorted item and run; false past the end of the queue
  __device__ __forceinline__ bool locate(int pos, int v, int* item, int* run) const {
    const int ir = (pos / nbr) * DMQ_XCDS + queue_of(v);
    if ((unsigned)ir >= (unsigned)n) return false;        // also a position from queue words that were not zero
    *item = order[ir];
    *run = pos - (pos / nbr) * nbr;
    return true;
  }
  __device__ __forceinline__ void fill(RowsUnit& u, const int4_t& r0, const int4_t& r1, int run) const {
    // the record is the same for every lane: scalar registers from here on (addresses built from
    // these fields then are a scalar base plus a lane offset)
    auto uni = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
    const int ttile = uni(r0[2]), tstart = uni(r0[3]), tcount = uni(r1[0]), gu_ss = uni(r1[1]);
    const int row0 = ttile * DMQ_ROWS_TILE;
    const int rows = min(tcount - row0, DMQ_ROWS_TILE);
    u.valid = 1;
    u.cls = rows > 64 ? 0 : (rows > 32 ? 1 : 2);
    u.pool = uni(r0[0]);
    u.kb0 = uni(run) * nbl;
    u.r_first = tstart + row0;
    u.r_end = tstart + tcount;
    u.slice_start = slice_is_groups ? uni(r1[2]) : gu_ss;
    u.post_slice = gu_ss / (2 * DMQ_GS);
  }
  // Draw a unit and wait for it (start of the kernel, change of class, end of the queues): own
  // queue first, then the others in XCD order.
  __device__ __forceinline__ void fetch_sync(RowsUnit& u) {
    u.valid = 0;
    while (victim < DMQ_XCDS) {
      if (threadIdx.x == 0)
        mail[0] = __hip_atomic_fetch_add(queue + queue_of(victim), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      const int pos = __builtin_amdgcn_readfirstlane(mail[0]) + wgs;
      __syncthreads();
      int item, run;
      if (DMQ_UNI(locate(pos, victim, &item, &run))) {
        item = __builtin_amdgcn_readfirstlane(item);
        const int4_t* rec = (const int4_t*)(items + (long)DMQ_ITEM_WORDS * item);
        fill(u, rec[0], rec[1], run);
        return;
      }
      ++victim;
    }
  }
};

template <int BIT, int TT, int EPI>
__device__ __forceinline__ void dmq_rows_body(const GemmParams& p, RowsSched& sc, RowsUnit& cur_io,
                                              int& lut_key, uint8_t* lds) {
  RowsUnit cur = cur_io.uniform();
  constexpr int MODE = DMQ_MODE_A16;
  constexpr int NT = 4;
  constexpr int WW = BIT;                                // packed words per lane, group and n-tile
  constexpr int PPG = DMQ_GS * BIT / 8;                  // packed bytes per weight row and group
  constexpr int AB = 256;                                // activation bytes per row and group
  constexpr int SLOT = 16 * TT * AB;
  constexpr bool SILU = (EPI == DMQ_EPI_SILU || EPI == DMQ_EPI_SILU_ROT);
  constexpr int FPB = SILU ? 128 : 256;                  // output features per block
  constexpr int CPT = TT;                                // 16-byte chunks a thread stages per group
  constexpr int DMA_STEP = (TT < 3) ? 2 : 3;             // MFMA step behind the barrier of a group step
  // Table rows of 256 bytes (the address of a look-up is one byte permute) where the three
  // activation buffers leave the room: up to 64 rows.  128-row units keep 128-byte rows.
  constexpr int ROW = (TT <= 4) ? 256 : DMQ_LUT_ROW;
  uint8_t* const tbl = lds;
  uint8_t* const stage = lds + 256 * ROW;

  // The kernel holds nine instances of this body in one loop.  The thread index goes through an
  // empty asm so that the lane constants below are computed here, per call: hoisted out of that
  // loop, the constants of all nine instances would be live at once and spill.
  int tidv = threadIdx.x;
  asm volatile("" : "+v"(tidv));
  const int lane = tidv & 63;
  const int wave = tidv >> 6;
  const int l16 = lane & 15;
  const int q = lane >> 4;
  const uint32_t lane_base = dmq_lut_lane_base<BIT, 2, ROW>(lane);
  // every unit of this call is of this pool and class (both the same for every lane)
  const int my_pool = __builtin_amdgcn_readfirstlane(cur.pool), my_cls = __builtin_amdgcn_readfirstlane(cur.cls);
  const PoolW& pw = p.pool[my_pool];
  const int G = p.groups;
  const int S = sc.nbl * G;                              // group steps of a unit
  const bool pipelined = S >= DMQ_ROWS_MIN_STEPS;        // shorter units: the next one is drawn afterwards

  // ---- lane offsets that do not depend on the unit
  uint32_t w_lane[NT], n_lane[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int wr = SILU ? ((j & 1) ? p.half_width : 0) + wave * 32 + (j >> 1) * 16 : wave * 64 + j * 16;
    w_lane[j] = (uint32_t)(wr + l16) * PPG + q * (WW * 4);
    n_lane[j] = (uint32_t)(wr + l16) * 2;
  }
  const long w_gstride = (long)pw.n_total * PPG;
  const long n_gstride = (long)pw.n_total * 2;
  // staging: load c of a wave covers four whole rows of the tile (16 lanes per row: the 256
  // contiguous bytes of the row's group); a thread stages chunk lane % 16 of rows
  // wave*4*TT + 4c + lane / 16.  Rows past the expert's last row stage a copy of that last row:
  // every load is unconditional and nothing computed from such a row is ever stored.
  // The load writes LDS lane by lane (lane L of load c: byte 16 L of the four rows), so the
  // swizzle is applied on the memory side: position lane % 16 of row r holds chunk
  // (lane % 16) ^ (r % 16) of that row, and that is the chunk the lane requests.
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const uint32_t stage_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)stage;
  // operand reads: row 16 t + l16, chunk (4 q + s) ^ l16
  uint32_t b_off[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) b_off[s] = (uint32_t)(l16 * AB + (((4 * q + s) ^ l16) * 16));

  // ---- load side: the unit whose operands are being requested (three group steps ahead)
  const uint8_t* Lw;
  const uint8_t* Ln;
  uint32_t a_lane[CPT];
  int lk = 0, lg = 0;                                    // weights: feature block and group of step + 3
  int ak = 0, ag = 0;                                    // activations: the same for step + 2
  int l_state = 0;                                       // 1: the weight loads are in the next unit, 2: held at the last step
  int a_frozen = 0;
  auto set_bases = [&](const RowsUnit& u) {
    const long g_base = p.slice_is_groups ? u.slice_start : 0;
    const long row0 = (p.slice_is_groups ? 0 : u.slice_start) + (long)u.kb0 * FPB;
    Lw = pw.w + (g_base * pw.n_total + row0) * PPG;
    Ln = (const uint8_t*)pw.norms + (g_base * pw.n_total + row0) * 2;
  };
  auto stage_rows = [&](const RowsUnit& u, int (&ri)[CPT]) {
    // (the first row goes through an empty asm: the per-chunk row numbers are cheap to recompute and
    // would otherwise be kept, and spilled, across the whole call)
    int row0 = wave * (4 * TT) + q;
    asm volatile("" : "+v"(row0));
    const int* const rix = pw.row_index;
    if (rix) {
#pragma unroll
      for (int c = 0; c < CPT; ++c) ri[c] = rix[min(u.r_first + row0 + c * 4, u.r_end - 1)];
    } else {
#pragma unroll
      for (int c = 0; c < CPT; ++c) ri[c] = min(u.r_first + row0 + c * 4, u.r_end - 1);
    }
  };
  auto lanes_from_rows = [&](const int (&ri)[CPT], uint32_t (&al)[CPT]) {
#pragma unroll
    for (int c = 0; c < CPT; ++c)
      al[c] = (uint32_t)ri[c] * (uint32_t)p.act_row_bytes + (uint32_t)((l16 ^ ((wave * (4 * TT) + c * 4 + q) & 15)) * 16);
  };

  float4_t acc[NT][TT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int t = 0; t < TT; ++t) acc[j][t] = (float4_t){0.f, 0.f, 0.f, 0.f};

  uint32_t pk[4][NT][WW];            // packed weights of four consecutive group steps
  uint32_t nh[4][NT];                // norm of the lane's weight row
  uint32_t raw[NT][4];               // looked-up operand words on their way to being scaled (one MFMA step)
  uint4_t aop[2][NT];                // scaled weight operands of the current / next MFMA step
  uint4_t bf[4];                     // activation operands, three micro-steps ahead of their MFMAs

  // every address is a workgroup-uniform base (scalar registers) plus a 32-bit lane offset; the
  // empty asm keeps the zero-extension of the offset next to the load, which is the form the
  // scalar-base addressing mode of global loads needs
  auto lane_off = [](uint32_t o) { asm volatile("" : "+v"(o)); return o; };
  const uint8_t* const act_p = pw.act;
  auto load_w = [&](int j, uint32_t (&d)[WW], uint32_t& n) {
    const uint8_t* wb = Lw + (long)lk * (FPB * PPG) + lg * w_gstride;
    const uint8_t* nb = Ln + (long)lk * (FPB * 2) + lg * n_gstride;
    dmq_load_words<WW>(wb + lane_off(w_lane[j]), d);
    n = *(const uint16_t*)(nb + lane_off(n_lane[j]));
  };
  // chunk c of the activation tile of the activation-side position, straight into LDS buffer buf_off
  auto load_a = [&](int c, uint32_t buf_off) {
    const uint32_t m0v = stage_lds + buf_off + (uint32_t)((wave_u * (4 * TT) + c * 4) * AB);
    const uint8_t* src = act_p + (long)ag * AB;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(m0v), "v"(a_lane[c]), "s"(src) : "m0");
  };
  // every vector memory operation issued before the last `younger` ones has completed
  auto wait_loads = [](auto nc) {
    constexpr int younger = decltype(nc)::value;
    static_assert(younger >= 0 && younger < 64, "6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(younger) : "memory");
  };
  auto look = [&](auto sc_, const uint32_t (&pkj)[WW], uint32_t (&w)[4]) {
    constexpr int s = decltype(sc_)::value;
    dmq_dequant_step<MODE, BIT, s, false, ROW>(tbl, lane_base, pkj, w);
  };
  auto read_b = [&](uint32_t buf_off, int s, int t) -> uint4_t {
    return *(const uint4_t*)(stage + buf_off + b_off[s] + t * (16 * AB));
  };

  // ---- the next unit, assembled while the current one runs
  RowsUnit nxt;
  nxt.valid = 0;
  int nxt_ready = 0;
  int pop_v = 0, nxt_run = 0;
  int4_t nrec0 = {0, 0, 0, 0}, nrec1 = {0, 0, 0, 0};
  int nxt_ri[CPT];                                       // row indices, then lane offsets of the next unit
#pragma unroll
  for (int c = 0; c < CPT; ++c) nxt_ri[c] = 0;
  int nxt_located = 0;
  // stage k runs at the top of group step k of every unit
  auto desc_stage = [&](int k) {
    if (k == 0) {
      nxt.valid = 0; nxt_ready = 0; nxt_located = 0;
      if (DMQ_UNI(sc.victim) < DMQ_XCDS && threadIdx.x == 0)
        pop_v = __hip_atomic_fetch_add(sc.queue + sc.queue_of(sc.victim), 1, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
    } else if (k == 1) {
      if (threadIdx.x == 0) sc.mail[0] = pop_v;         // visible after this step's barrier
    } else if (k == 2) {
      if (DMQ_UNI(sc.victim) < DMQ_XCDS) {
        const int pos = __builtin_amdgcn_readfirstlane(sc.mail[0]) + sc.wgs;
        int item;
        if (DMQ_UNI(sc.locate(pos, sc.victim, &item, &nxt_run))) {
          item = __builtin_amdgcn_readfirstlane(item);
          const int4_t* rec = (const int4_t*)(sc.items + (long)DMQ_ITEM_WORDS * item);
          nrec0 = rec[0]; nrec1 = rec[1];
          nxt_located = 1;
        } else {
          ++sc.victim;                                   // this queue is empty: the next draw waits
        }
      }
    } else if (k == 3) {
      if (DMQ_UNI(nxt_located)) {
        sc.fill(nxt, nrec0, nrec1, nxt_run);
        if (nxt.cls == my_cls && nxt.pool == my_pool) stage_rows(nxt, nxt_ri);
      }
    } else {
      if (DMQ_UNI(nxt.valid && nxt.cls == my_cls && nxt.pool == my_pool)) {
#pragma unroll
        for (int c = 0; c < CPT; ++c)
          nxt_ri[c] = (int)((uint32_t)nxt_ri[c] * (uint32_t)p.act_row_bytes +
                            (uint32_t)((l16 ^ ((wave * (4 * TT) + c * 4 + q) & 15)) * 16));
        nxt_ready = 1;
      }
    }
  };
  auto advance_load = [&]() {
    if (DMQ_UNI(l_state) == 2) return;
    if (++lg == G) {
      lg = 0;
      if (++lk == sc.nbl) {
        const int go_on = DMQ_UNI(nxt_ready);            // the stream goes on with the next unit,
        l_state = go_on ? 1 : 2;                         // or repeats the last step of this one
        if (go_on) {
          set_bases(nxt.uniform());
          lk = 0;
        } else {
          lk = sc.nbl - 1; lg = G - 1;
        }
      }
    }
  };
  auto advance_act = [&]() {                             // the same walk, one step behind
    if (DMQ_UNI(a_frozen)) return;
    if (++ag == G) {
      ag = 0;
      if (++ak == sc.nbl) {
        if (DMQ_UNI(nxt_ready)) {
#pragma unroll
          for (int c = 0; c < CPT; ++c) a_lane[c] = (uint32_t)nxt_ri[c];
          ak = 0;
        } else {
          ak = sc.nbl - 1; ag = G - 1;
          a_frozen = 1;
        }
      }
    }
  };

  // ---- empty pipeline: table, steps 0..2 of the weights, activation tiles 0 and 1 in LDS
  {
    int ri[CPT];
    stage_rows(cur, ri);
    set_bases(cur);
    uint32_t lutw[4];
    const int my_key = cur.pool * 2 + (ROW == 256 ? 1 : 0);   // the table in LDS: pool and row size
    const bool build = __builtin_amdgcn_readfirstlane(lut_key) != my_key;
    if (build) dmq_lut_fetch<BIT, 2>(pw.lut, threadIdx.x, lutw);
    lanes_from_rows(ri, a_lane);
#pragma unroll
    for (int c = 0; c < CPT; ++c) load_a(c, 0);
#pragma unroll
    for (int j = 0; j < NT; ++j) load_w(j, pk[0][j], nh[0][j]);
    lg = 1; ag = 1;
#pragma unroll
    for (int c = 0; c < CPT; ++c) load_a(c, SLOT);
#pragma unroll
    for (int j = 0; j < NT; ++j) load_w(j, pk[1][j], nh[1][j]);
    lg = 2; ag = 2;
#pragma unroll
    for (int j = 0; j < NT; ++j) load_w(j, pk[2][j], nh[2][j]);
    lg = 3;
    if (build) {
      __syncthreads();                                   // nobody reads the old table any more
      dmq_lut_store_wave<BIT, 2, ROW>(tbl, wave, lutw);
      lut_key = my_key;
    }
    wait_loads(std::integral_constant<int, 0>{});        // both tiles have landed
    __syncthreads();
  }
  uint32_t cur_off = 0, nxt_off = SLOT, wr_off = 2 * SLOT;
  auto scale_words = [](const uint32_t (&w)[4], uint32_t nword) -> uint4_t {
    const half2_t nn = __builtin_bit_cast(half2_t, nword);
    uint4_t r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, w[i]) * nn);
    return r;
  };
  auto splat = [](uint32_t n16) -> uint32_t { return (n16 & 0xffffu) * 0x10001u; };
  // pipeline state at the head of a group step: scaled operands of MFMA step 0, looked-up words of
  // step 1, activation operands of micro-steps 0..2
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    uint32_t r0[4];
    look(std::integral_constant<int, 0>{}, pk[0][j], r0);
    aop[0][j] = scale_words(r0, splat(nh[0][j]));
    look(std::integral_constant<int, 1>{}, pk[0][j], raw[j]);
  }
#pragma unroll
  for (int m = 0; m < 3; ++m) bf[m] = read_b(cur_off, m / TT, m % TT);

  // scatter epilogue: routing weight and destination row of the lane's rows, requested when the
  // unit starts
  float row_w[TT];
  int row_dst[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) { row_w[t] = 0.f; row_dst[t] = 0; }
  int kb = cur.kb0;                                      // feature block in progress

  // ---- store the finished block kb of the current unit
  auto epilogue = [&]() {
    int rlog[TT];
    bool avalid[TT];
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      rlog[t] = cur.r_first + t * 16 + l16;
      avalid[t] = rlog[t] < cur.r_end;
    }
    const int feat_k = kb * FPB + wave * (FPB / 4);      // first output feature of the wave
    if constexpr (EPI == DMQ_EPI_STORE) {
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        if (!avalid[t]) continue;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          const half4_t h = {(_Float16)acc[j][t][0], (_Float16)acc[j][t][1], (_Float16)acc[j][t][2],
                             (_Float16)acc[j][t][3]};
          *(half4_t*)(p.out + (long)rlog[t] * p.out_stride + feat_k + j * 16 + 4 * q) = h;
        }
      }
    } else if constexpr (EPI == DMQ_EPI_SCATTER) {
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        if (!avalid[t]) continue;
        __half* orow = p.out_slots + (long)row_dst[t] * p.out_stride + feat_k + 4 * q;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          const float4_t v = acc[j][t] * row_w[t];
          const half4_t h = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
          *(half4_t*)(orow + j * 16) = h;
        }
      }
    } else if constexpr (EPI == DMQ_EPI_SILU) {
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        if (!avalid[t]) continue;
#pragma unroll
        for (int j = 0; j < NT; j += 2) {
          half4_t h;
#pragma unroll
          for (int r = 0; r < 4; ++r) h[r] = (_Float16)(dmq_silu(acc[j][t][r]) * acc[j + 1][t][r]);
          *(half4_t*)(p.out + (long)rlog[t] * p.out_stride + feat_k + (j >> 1) * 16 + 4 * q) = h;
        }
      }
    } else {
      // SiLU * up rows of the block (one group of the down projection) -> rotation of that group by
      // the expert's matrix -> fp16 rows.  The tile meets in the LDS buffer of the finished step
      // (once every wave is done reading it: a barrier), every wave rotates it onto 32 of the 128
      // outputs with its quarter of the matrix: the arithmetic of the stand-alone rotation kernel,
      // in its order.  The buffer is next written behind the following step's barrier.
      constexpr int PITCH = 256;
      const int blk = kb * FPB;
      uint8_t* tile = stage + wr_off;
      const __half* prot = pw.post_rot + (long)(cur.post_slice + blk / DMQ_GS) * (DMQ_GS * DMQ_GS) +
                           (long)(32 * wave + l16) * DMQ_GS + 8 * q;
      __syncthreads();
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        const int row = t * 16 + l16;
#pragma unroll
        for (int j = 0; j < NT; j += 2) {
          half4_t h;
#pragma unroll
          for (int r = 0; r < 4; ++r) h[r] = (_Float16)(dmq_silu(acc[j][t][r]) * acc[j + 1][t][r]);
          const int f = 32 * wave + (j >> 1) * 16 + 4 * q;
          const int c = f >> 3;
          *(half4_t*)(tile + row * PITCH + ((c ^ (row & 15)) * 16) + (f & 7) * 2) = h;
        }
      }
      __syncthreads();
      const int col0 = blk + 32 * wave + 4 * q;
      // the wave's two output tiles one after the other (half the registers; the tile is read twice)
#pragma unroll
      for (int jt = 0; jt < 2; ++jt) {
        uint4_t pa[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) pa[s] = *(const uint4_t*)(prot + (long)jt * 16 * DMQ_GS + 32 * s);
        float4_t racc[TT];
#pragma unroll
        for (int t = 0; t < TT; ++t) racc[t] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 4; ++s) {
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            const int row = t * 16 + l16;
            const uint4_t braw = *(const uint4_t*)(tile + row * PITCH + (((4 * s + q) ^ (row & 15)) * 16));
            racc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, pa[s]),
                                                             __builtin_bit_cast(half8_t, braw), racc[t], 0, 0, 0);
          }
        }
#pragma unroll
        for (int t = 0; t < TT; ++t) {
          if (!avalid[t]) continue;
          uint8_t* orow = p.post_out + (long)rlog[t] * p.post_row_bytes;
          const half4_t h = {(_Float16)racc[t][0], (_Float16)racc[t][1], (_Float16)racc[t][2], (_Float16)racc[t][3]};
          *(half4_t*)(orow + (col0 + 16 * jt) * 2) = h;
        }
      }
    }
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int t = 0; t < TT; ++t) acc[j][t] = (float4_t){0.f, 0.f, 0.f, 0.f};
    ++kb;
  };

  // ---- one group step: GI = st % 4 selects the register ring entries at compile time.
  // A group is 4 * TT micro-steps (MFMA step s, row tile t) of four MFMAs each (the wave's four
  // n-tiles against one activation operand).  A wave issues in order, so matrix and vector work
  // only overlap when they alternate in the instruction stream: between its MFMAs a micro-step
  // carries the activation operand of three micro-steps later, and for the n-tiles assigned to it
  // the scaling of the next MFMA step's looked-up words and the look-ups of the step after that,
  // plus its share of the step's global loads and LDS stores.  Nothing of it feeds its own MFMAs.
  auto group = [&](auto gic, int st) {
    constexpr int GI = decltype(gic)::value;
    if (pipelined) {                          // the next unit is drawn while this one runs
      if (st == GI) desc_stage(GI);
      if (GI == 0 && st == 4) desc_stage(4);
    }
    if constexpr (EPI == DMQ_EPI_SCATTER) {
      if (GI == 0 && st == 0) {
#pragma unroll
        for (int t = 0; t < TT; ++t) {
          const int rr = min(cur.r_first + t * 16 + l16, cur.r_end - 1);
          row_w[t] = p.row_weight[rr];
          row_dst[t] = p.row_slot[rr];
        }
      }
    }
    uint32_t n2c[NT], n2n[NT];                // norms of this step's and the next step's weight rows
#pragma unroll
    for (int j = 0; j < NT; ++j) { n2c[j] = splat(nh[GI][j]); n2n[j] = splat(nh[(GI + 1) & 3][j]); }
    auto micro = [&](auto sc_, auto tc) {
      constexpr int s = decltype(sc_)::value, t = decltype(tc)::value;
      constexpr int m = s * TT + t;
      {
        constexpr int m3 = m + 3;
        if constexpr (m3 < 4 * TT) bf[m3 & 3] = read_b(cur_off, m3 / TT, m3 % TT);
        else bf[m3 & 3] = read_b(nxt_off, (m3 - 4 * TT) / TT, (m3 - 4 * TT) % TT);
      }
      const half8_t b = __builtin_bit_cast(half8_t, bf[m & 3]);
#pragma unroll
      for (int j = 0; j < NT; ++j)
        acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, aop[s & 1][j]), b,
                                                           acc[j][t], 0, 0, 0);
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        if ((j * TT) / NT != t) continue;
        aop[(s + 1) & 1][j] = scale_words(raw[j], s + 1 < 4 ? n2c[j] : n2n[j]);
        if constexpr (s + 2 < 4) look(std::integral_constant<int, (s + 2) & 3>{}, pk[GI][j], raw[j]);
        else look(std::integral_constant<int, (s + 2) & 3>{}, pk[(GI + 1) & 3][j], raw[j]);
        if constexpr (s == 1) load_w(j, pk[(GI + 3) & 3][j], nh[(GI + 3) & 3][j]);   // three steps ahead
      }
      // the activation tile of step st + 2, into the buffer the previous step has read: requested
      // behind the barrier of this step, which every wave passes only when it is done with that one
      if constexpr (s == DMA_STEP) load_a(t, wr_off);
    };
    // The issue order inside an MFMA step: a wave alone on its SIMD issues at most one instruction
    // every four cycles and an MFMA keeps the matrix pipe for sixteen, so up to three other
    // instructions fit behind each MFMA for free, and none of this step's other work depends on
    // this step's MFMAs: one MFMA, then up to three vector / scalar / LDS / memory instructions.
    auto mfma_step = [&](auto sc_) {
      micro(sc_, std::integral_constant<int, 0>{});
      micro(sc_, std::integral_constant<int, 1>{});
      if constexpr (TT > 2) {
        micro(sc_, std::integral_constant<int, 2>{});
        micro(sc_, std::integral_constant<int, 3>{});
      }
      if constexpr (TT > 4) {
        micro(sc_, std::integral_constant<int, 4>{});
        micro(sc_, std::integral_constant<int, 5>{});
        micro(sc_, std::integral_constant<int, 6>{});
        micro(sc_, std::integral_constant<int, 7>{});
      }
#pragma unroll
      for (int i = 0; i < 4 * TT; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x326, TT >= 8 ? 3 : (TT == 4 ? 5 : 10), 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    // One barrier per step.  The last three micro-steps of a step already read operands of the
    // next step's tile, so the barrier stands inside the step: in front of MFMA step 3 (with two
    // row tiles MFMA step 2 holds one of those micro-steps: in front of that).  It publishes the
    // next step's tile, requested behind the previous step's barrier (since then this wave has
    // issued the 8 weight loads of this step, in MFMA step 1, and nothing else), and a wave that
    // has passed it knows every wave done with the previous step, whose buffer takes the tile after
    // next.
    auto publish_next_tile = [&]() {
      wait_loads(std::integral_constant<int, 8>{});
      __syncthreads();
    };
    mfma_step(std::integral_constant<int, 0>{});
    mfma_step(std::integral_constant<int, 1>{});
    if constexpr (TT < 3) publish_next_tile();
    mfma_step(std::integral_constant<int, 2>{});
    if constexpr (TT >= 3) publish_next_tile();
    mfma_step(std::integral_constant<int, 3>{});
    advance_load();
    advance_act();
    const uint32_t o = cur_off; cur_off = nxt_off; nxt_off = wr_off; wr_off = o;
  };


  int gcount = 0;                                        // groups of the block in progress that are done
  for (;;) {
    for (int st = 0; st < S; st += 4) {
      group(std::integral_constant<int, 0>{}, st);
      group(std::integral_constant<int, 1>{}, st + 1);
      group(std::integral_constant<int, 2>{}, st + 2);
      group(std::integral_constant<int, 3>{}, st + 3);
      gcount += 4;
      if (gcount == G) { epilogue(); gcount = 0; }
    }
    if (DMQ_UNI(l_state) != 1) break;
    cur = nxt.uniform();                                 // its first three steps are already on their way
    kb = cur.kb0;
    l_state = 0;
  }
  // tile loads of the last steps are still on their way to LDS buffers that the next call lays
  // out differently
  wait_loads(std::integral_constant<int, 0>{});
  // the unit after this call: the one already drawn (another class or pool), or a fresh draw
  if (DMQ_UNI(nxt.valid)) cur_io = nxt;
  else sc.fetch_sync(cur_io);
}

// One workgroup per CU; see the head of the file.  Pools of another mode or of 8-bit indices are
// skipped (they belong to dmq_gemm_gf_kernel launches over the same list).
template <int EPI>
__global__ __launch_bounds__(256) void dmq_gemm_rows_kernel(GemmParams p, int* queue, int nbl) {
  extern __shared__ __attribute__((aligned(16))) uint8_t dmq_rows_lds[];
  uint8_t* stage = dmq_rows_lds + DMQ_LUT_BYTES;         // scratch of the sort below
  uint16_t* order = (uint16_t*)(dmq_rows_lds + DMQ_ROWS_ORDER_OFF);
  int* mail = (int*)(dmq_rows_lds + DMQ_ROWS_MAIL_OFF);
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;

  // ---- the work items in order of tile class (stable inside a class): every workgroup sorts the
  // list for itself, one round trip for the records and a scan
  const int n_items = min(p.n_items[0], DMQ_ROWS_MAX_ITEMS);
  const int ipt = (n_items + 255) >> 8;                  // items per thread, contiguous
  constexpr int IPT_MAX = DMQ_ROWS_MAX_ITEMS / 256;
  // which pools this launch serves (fp16 activations, 1/2/4-bit indices), one bit per pool
  unsigned elig = 0;
#pragma unroll
  for (int q = 0; q < DMQ_MAX_POOLS; ++q)
    elig |= (p.pool[q].mode == DMQ_MODE_A16 && p.pool[q].bit != 8) ? 1u << q : 0u;
  // all records are requested before any is looked at (positions past the list repeat its last
  // record: the loads are unconditional)
  int rpool[IPT_MAX], rtile[IPT_MAX], rcount[IPT_MAX];
#pragma unroll
  for (int k = 0; k < IPT_MAX; ++k) {
    rpool[k] = 0; rtile[k] = 0; rcount[k] = 0;
    if (k < ipt) {                                       // uniform
      const int i = max(min(tid * ipt + k, n_items - 1), 0);
      const int4_t r0 = *(const int4_t*)(p.items + (long)DMQ_ITEM_WORDS * i);
      rpool[k] = r0[0]; rtile[k] = r0[2];
      rcount[k] = p.items[(long)DMQ_ITEM_WORDS * i + 4];
    }
  }
  int cls[IPT_MAX];
  unsigned long long cnt = 0;                            // three 16-bit counters
#pragma unroll
  for (int k = 0; k < IPT_MAX; ++k) {
    cls[k] = 3;
    const int i = tid * ipt + k;
    const int rows = rcount[k] - rtile[k] * DMQ_ROWS_TILE;
    if (k < ipt && i < n_items && rows > 0 && ((elig >> (rpool[k] & (DMQ_MAX_POOLS - 1))) & 1u)) {
      cls[k] = rows > 64 ? 0 : (rows > 32 ? 1 : 2);
      cnt += 1ull << (16 * cls[k]);
    }
  }
  unsigned long long incl = cnt;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const unsigned lo = __shfl_up((unsigned)incl, d, 64);
    const unsigned hi = __shfl_up((unsigned)(incl >> 32), d, 64);
    if (lane >= d) incl += ((unsigned long long)hi << 32) | lo;
  }
  unsigned long long* wsum = (unsigned long long*)stage;  // [4]
  if (lane == 63) wsum[wave] = incl;
  __syncthreads();
  unsigned long long before = incl - cnt, total = 0;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const unsigned long long v = wsum[w];
    if (w < wave) before += v;
    total += v;
  }
  const int tot0 = (int)(total & 0xffff), tot1 = (int)((total >> 16) & 0xffff), tot2 = (int)((total >> 32) & 0xffff);
  int at[3] = {(int)(before & 0xffff), tot0 + (int)((before >> 16) & 0xffff),
               tot0 + tot1 + (int)((before >> 32) & 0xffff)};
#pragma unroll
  for (int k = 0; k < IPT_MAX; ++k) {
    if (cls[k] < 3) {
      const int c = cls[k];
      const int pos = c == 0 ? at[0]++ : (c == 1 ? at[1]++ : at[2]++);
      order[pos] = (uint16_t)(tid * ipt + k);
    }
  }
  __syncthreads();

  RowsSched sc;
  sc.queue = queue; sc.items = p.items; sc.order = order; sc.mail = mail;
  sc.n = tot0 + tot1 + tot2;
  sc.nbl = nbl; sc.nbr = p.n_blocks / nbl;
  sc.wgs = gridDim.x / DMQ_XCDS;
  sc.xcd = blockIdx.x % DMQ_XCDS;
  sc.victim = 0;
  sc.slice_is_groups = p.slice_is_groups;

  // the first unit of every workgroup is fixed: position (workgroup index inside the XCD) of its
  // own queue; the queue words count the positions drawn beyond those
  RowsUnit cur;
  cur.valid = 0;
  {
    int item, run;
    if (sc.locate(blockIdx.x / DMQ_XCDS, 0, &item, &run)) {
      item = __builtin_amdgcn_readfirstlane(item);
      const int4_t* rec = (const int4_t*)(p.items + (long)DMQ_ITEM_WORDS * item);
      sc.fill(cur, rec[0], rec[1], run);
    } else {
      sc.fetch_sync(cur);
    }
  }
  int lut_key = -1;
  while (cur.valid) {
    const int bit = p.pool[cur.pool].bit;
#define DMQ_ROWS_CALL(BIT, TT) dmq_rows_body<BIT, TT, EPI>(p, sc, cur, lut_key, dmq_rows_lds)
#define DMQ_ROWS_BIT(TT) \
    if (bit == 1) DMQ_ROWS_CALL(1, TT); else if (bit == 2) DMQ_ROWS_CALL(2, TT); else DMQ_ROWS_CALL(4, TT);
    if (cur.cls == 0) { DMQ_ROWS_BIT(8) }
    else if (cur.cls == 1) { DMQ_ROWS_BIT(4) }
    else { DMQ_ROWS_BIT(2) }
#undef DMQ_ROWS_BIT
#undef DMQ_ROWS_CALL
    __syncthreads();                                     // the next body starts with a fresh pipeline
  }
  // the last workgroup to leave puts the queue words back to zero for the next launch
  if (tid == 0) {
    const int left = __hip_atomic_fetch_add(queue + DMQ_XCDS, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (left == (int)gridDim.x - 1) {
#pragma unroll
      for (int i = 0; i <= DMQ_XCDS; ++i)
        __hip_atomic_store(queue + i, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}
