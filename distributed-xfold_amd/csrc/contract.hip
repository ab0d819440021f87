// Triangle contraction on bf16 MFMA:  T[c][i][j] = sum_k A[c][i][k] * B[c][j][k]
// for a batch of channels c, bf16 in and out, fp32 accumulation.  The same
// kernel, with a per-column or SwiGLU epilogue, takes the large dense
// projections (x W^T with thousands of rows and columns) of the diffusion
// transformer and the outer-product mean.
//
// Both operands are k-contiguous (the natural fragment order of
// v_mfma_f32_32x32x16_bf16).  The tile is as large as the register file
// allows: one workgroup of four waves per CU, a 256x256 block, each wave a
// 128x128 quadrant = 4x4 MFMA tiles = 256 fp32 accumulators (the unified
// 512-entry register file of a lone wave per SIMD), half a 16-byte fragment
// read per MFMA and 128 FLOPs per byte fetched from L2.
//
// What paces the kernel is the CU's vector memory path: every 64-byte row piece of a slab
// is a miss in the CU's L1 and a round trip to L2 (about 450 cycles on average with a
// quarter of them going on to memory), the L1 holds a limited number of them in flight, and
// a wave that issues a load into a full queue stalls with its MFMAs behind it.  A lone wave
// per SIMD has nobody to cover for it.  So:
//   * slabs (32 k deep) go from global memory straight into LDS
//     (global_load_lds_dwordx4: no staging registers, no LDS stores in the
//     instruction stream);
//   * the loads are spread evenly, one per four MFMAs per wave, which keeps the
//     memory path evenly busy instead of saturated in bursts;
//   * four LDS buffers: a load is issued two to three slabs (2000-3000 cycles)
//     before anybody waits for it, about the latency of a miss that goes to HBM;
//   * the one barrier per slab sits between its two k-steps, after the wave has
//     read all its fragments of the slab: the MFMAs of the second k-step cover
//     the barrier and the first fragment reads of the next slab, and the
//     buffer is free for refill the moment the barrier is passed;
//   * the workgroups are persistent, one per CU, and the slab pipeline never drains: the
//     loads that run ahead of a tile's last slabs fetch the first slabs of the
//     workgroup's next tile, the epilogue stages through an LDS area of its own and does
//     not wait for its stores, so a tile's first slab is in LDS when the previous tile's
//     last store has been issued.
// A load puts lane l's 16 bytes at LDS base + 16 l, so rows cannot be padded;
// instead the four 16-byte chunks of a 64-byte row are permuted, chunk c of row
// r living at position c ^ ((r >> 2) & 3), which makes the fragment reads (32
// rows x one chunk per half-wave) conflict-free over the 64 banks.  The
// permutation is applied on the global side, where a lane is free to fetch
// any chunk.
//
// The accumulators hold T^T tiles (B fragments as the MFMA's A operand), so a
// lane owns one output row i and four consecutive columns j per register quad:
// the epilogue packs those to 8 bytes, stages 32 rows x 64 columns at a time per wave
// through LDS and writes 128-byte row segments.
#include <algorithm>
#include <type_traits>

#include "common.h"
#include "kernels.h"

namespace {

// The block is 64 IT x 256: IT = 4 MFMA tiles per wave along i (256 x 256), or IT = 3 (192 x 256) where
// that saves enough rounds of workgroups (N = 384: tiles of 256 would be half empty).
constexpr int CN = 256, CK = 32;
constexpr int ROWB = CK * 2;            // bytes of a slab row in LDS (unpadded)
constexpr int SLAB = (256 + CN) * ROWB;  // 32 KB at IT = 4: A rows first, then B rows
constexpr int LDE = 64 + 8;             // LDS row stride of a wave's output staging area (bf16)
constexpr int EPI_BYTES = 32 * LDE * 2;  // 32 rows x 64 columns per wave at a time
constexpr int RSRC_RAW = 0x00020000;     // last word of a raw (unstructured, range-checked) buffer descriptor

// 64 lanes x 16 bytes from global (uniform base + per-lane byte offset) to
// 1 KB of LDS starting at the wave-uniform address dst.  Issued as inline assembly on purpose:
// the compiler keeps a scoreboard of the loads into LDS that it can see and, where paths with
// different waits meet, makes a later fragment read wait for ALL of them (vmcnt(0)), the ones
// issued a moment ago for slabs far ahead included.  Here every buffer is read only after an
// explicit wait and barrier that follow the load's issue.
__device__ __forceinline__ void load_to_lds(const char* base, uint32_t off, const char* dst) {
  const uint32_t lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)dst;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(off), "s"(base) : "m0");
}

// a pointer the compiler cannot prove wave-uniform, moved to scalar registers
template <typename T>
__device__ __forceinline__ T* uniform_ptr(T* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return reinterpret_cast<T*>(((uint64_t)hi << 32) | lo);
}

// One accumulator value, read where the source says: left to itself the register allocator,
// faced with an epilogue of many basic blocks, copies most of the 256 accumulators out of their
// accumulation registers up front, which costs as many vector registers (and spills).
__device__ __forceinline__ float acc_read(float a) {
  float v;
  asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
  return v;
}

// s_waitcnt with vmcnt = n, lgkmcnt = 0 (expcnt left alone)
template <int N>
__device__ __forceinline__ void wait_loads_but() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x70);
}

// MODE 0: plain bf16 product (the triangle contraction).
// MODE 1: per-column epilogue of the dense projections, (acc + bias) * alpha
//         and / or a sigmoid, uniform over the tile or chosen per segment of
//         seg_len columns, and optionally the 32x32-regrouped output order.
// MODE 2: SwiGLU, weight rows packed in blocks of 64 (32 "a" rows, then the 32
//         matching "b" rows): output column 32 p + x = silu(a) * b of block p.
enum { BIG_PLAIN = 0, BIG_COLUMN_OPS = 1, BIG_SWIGLU = 2 };

template <int MODE, int IT = 4>
__global__ __launch_bounds__(256, 1) void contract_kernel(GemmArgs g) {
  constexpr int CM = 64 * IT, WM = 32 * IT;  // block and wave extent along i
  constexpr int SLAB_A = CM * ROWB;
  constexpr int NLOAD = IT + 4;              // loads per wave and slab
  constexpr int NSTORE = (MODE == BIG_SWIGLU ? 4 : 8) * IT;  // stores per wave and full tile
  static_assert(2 * NLOAD + IT + NSTORE < 64, "vmcnt has six bits");
  // four slab buffers and the waves' output staging areas
  __shared__ __attribute__((aligned(1024))) char sb0[SLAB];
  __shared__ __attribute__((aligned(1024))) char sb1[SLAB];
  __shared__ __attribute__((aligned(1024))) char sb2[SLAB];
  __shared__ __attribute__((aligned(1024))) char sb3[SLAB];
  __shared__ __attribute__((aligned(16))) char sOut[4 * EPI_BYTES];
  __shared__ __attribute__((aligned(16))) float sColBias[MODE == BIG_COLUMN_OPS ? 4 * 128 : 4];  // a wave's 128 bias values
  auto buf = [&](int i) -> char* { return (i & 3) == 0 ? sb0 : (i & 3) == 1 ? sb1 : (i & 3) == 2 ? sb2 : sb3; };

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hh = lane >> 5, l31 = lane & 31;
  const int wm = (wave >> 1) * WM, wn = (wave & 1) * 128;

  // The workgroups are persistent (one per CU) and walk their tiles in a fixed order.
  // XCD-aware mapping: workgroup ids are dealt round-robin to the 8 XCDs, so
  // id -> (xcd, slot) -> logical id makes each XCD walk a contiguous range of
  // (channel, j-tile, i-tile), i-tile fastest: the tiles that share a channel's
  // A and B panels run on one XCD at about the same time and find them in its L2.
  const int tiles_m = (g.M + CM - 1) / CM, tiles_n = (g.N + CN - 1) / CN;
  const int total = tiles_m * tiles_n * g.batch;
  const int per_xcd = (total + 7) / 8;
  const int xcd = blockIdx.x & 7, slot_step = gridDim.x >> 3;
  // One large product: an XCD that walks whole columns of tiles re-reads all of
  // A for every column, and A (8 MB at 4096 x 1024) does not stay in its 4 MB
  // L2.  Deal the XCDs a 4 x 2 grid of rectangles instead: a quarter of A stays
  // resident while the XCD streams through its half of B once.
  const bool rect = g.batch == 1 && (tiles_m & 3) == 0 && (tiles_n & 1) == 0;
  struct Tile { int m0, n0, bz; };
  auto tile_at = [&](int slot, Tile& t) -> bool {
    const int logical = xcd * per_xcd + slot;
    if (slot >= per_xcd || logical >= total) return false;
    int tm = logical % tiles_m, tn = (logical / tiles_m) % tiles_n;
    t.bz = logical / (tiles_m * tiles_n);
    if (rect) {
      const int mq = tiles_m >> 2, nh = tiles_n >> 1;
      tm = (xcd & 3) * mq + slot % mq;
      tn = (xcd >> 2) * nh + slot / mq;
    }
    // (the divisions above go through the vector unit; say again that the results are uniform)
    t.m0 = __builtin_amdgcn_readfirstlane(tm * CM);
    t.n0 = __builtin_amdgcn_readfirstlane(tn * CN);
    t.bz = __builtin_amdgcn_readfirstlane(t.bz);
    return true;
  };
  int slot = blockIdx.x >> 3;
  Tile cur_t, next_t;
  if (!tile_at(slot, cur_t)) return;

  // Per slab a wave issues IT loads for A and four for B: load i covers rows
  // 16 IT wave + 16 i .. + 16 of A, 64 wave + 16 i .. + 16 of B (one 64-byte row per 4 lanes).  The lane at position
  // pc of row r fetches chunk pc ^ ((r >> 2) & 3) = pc ^ (lane >> 4).  Rows past
  // the end repeat the last one (what they produce lands in output rows that
  // are never stored or in columns N..ldc-1 of T, which no consumer reads); a
  // chunk past K is fetched from the row's first slab instead and zeroed in
  // LDS before the slab is used.
  const int ld_r = lane >> 2;
  const int ld_c = (lane & 3) ^ (lane >> 4);
  const char* A;
  const char* B;
  uint32_t offa[4], offb[4];
  auto point_a = [&](const Tile& t) {
    A = reinterpret_cast<const char*>(g.A + (int64_t)t.bz * g.sA);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      offa[i] = ((uint32_t)min(t.m0 + 16 * IT * wave + 16 * i + ld_r, g.M - 1) * (uint32_t)g.lda + ld_c * 8) * 2u;
  };
  auto point_b = [&](const Tile& t) {
    B = reinterpret_cast<const char*>(g.B + (int64_t)t.bz * g.sB);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      offb[i] = ((uint32_t)min(t.n0 + 64 * wave + 16 * i + ld_r, g.N - 1) * (uint32_t)g.ldb + ld_c * 8) * 2u;
  };
  point_a(cur_t);
  point_b(cur_t);
  // Load i of half a slab: `first` = the wave's loads of A, else its four of B, of slab kt of the
  // tile that A / B point at.
  auto slab_load_one = [&](char* dst, int kt, bool first, int i) {
    const int k0 = kt * CK;
    const uint32_t kb = k0 + ld_c * 8 < g.K ? (uint32_t)k0 * 2u : 0u;
    if (first) load_to_lds(A, offa[i] + kb, dst + (16 * IT * wave + 16 * i) * ROWB);
    else load_to_lds(B, offb[i] + kb, dst + SLAB_A + (64 * wave + 16 * i) * ROWB);
  };
  auto slab_load = [&](char* dst, int kt, bool first) {
#pragma unroll
    for (int i = 0; i < (first ? IT : 4); ++i) slab_load_one(dst, kt, first, i);
  };
  // Chunks at or past K of slab kt (the last slab, and the all-zero slabs that
  // pad the slab count to a multiple of four): thread t clears them in row t
  // of A and row t of B.  Every wave's loads of the slab must have landed.
  auto slab_clear_tail = [&](char* b, int kt) {
    const int valid = max(0, min(4, (g.K - kt * CK) >> 3));
    const u32x4 z = {0, 0, 0, 0};
    const int swz = (tid >> 2) & 3;
    for (int c = valid; c < 4; ++c) {
      if (tid < CM) *reinterpret_cast<u32x4*>(b + tid * ROWB + ((c ^ swz) << 4)) = z;
      *reinterpret_cast<u32x4*>(b + SLAB_A + tid * ROWB + ((c ^ swz) << 4)) = z;
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  };

  // Fragment (row R = base + 32 t + l31, k-step ks, half hh) is chunk 2 ks + hh
  // of row R, at position (2 ks + hh) ^ ((R >> 2) & 3); the bases are multiples
  // of 32, so the permutation depends on l31 only.
  uint32_t fo[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) fo[ks] = (uint32_t)(l31 * ROWB + (((2 * ks + hh) ^ ((l31 >> 2) & 3)) << 4));
  const uint32_t a_base = (uint32_t)(wm * ROWB), b_base = (uint32_t)(SLAB_A + wn * ROWB);

  // acc[jt][it] = (T^T) tile: rows j = wn + 32 jt + .., columns i = wm + 32 it + ..
  f32x16 acc[4][IT];

  bf16x8 fa[2][IT], fb[2][4];  // set 0: first k-step of a slab, set 1: second
  auto frag = [&](int set, const char* b, int ks, int j) {
    if (j < IT) fa[set][j] = as_frag(*reinterpret_cast<const u32x4*>(b + a_base + j * (32 * ROWB) + fo[ks]));
    else fb[set][j - IT] = as_frag(*reinterpret_cast<const u32x4*>(b + b_base + (j - IT) * (32 * ROWB) + fo[ks]));
  };
  auto frags = [&](int set, const char* b, int ks) {
#pragma unroll
    for (int j = 0; j < IT + 4; ++j) frag(set, b, ks, j);
  };
  // The IT + 4 fragment reads of a k-step with half a slab's loads dealt evenly between them, in
  // this order in the source: the loads are opaque to the scheduler, which keeps memory
  // operations on their side of one, so this is what spreads the loads over the k-step.
  auto frags_and_loads = [&](int set, const char* b, int ks, char* dst, int kt, bool first) {
    const int nl = first ? IT : 4;
#pragma unroll
    for (int j = 0; j < IT + 4; ++j) {
      frag(set, b, ks, j);
      if (((j + 1) * nl) / (IT + 4) > (j * nl) / (IT + 4)) slab_load_one(dst, kt, first, (j * nl) / (IT + 4));
    }
  };
  // `fresh`: the first k-step of a tile starts its accumulators from the constant zero
  auto mfmas = [&](int set, auto fresh_c) {
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
#pragma unroll
      for (int it = 0; it < IT; ++it)
        acc[jt][it] = mfma32(fb[set][jt], fa[set][it], decltype(fresh_c)::value ? zero : acc[jt][it]);
  };
  // 4 IT MFMAs with the IT + 4 fragment reads (and the loads that sit between them) spread over them
  auto interleave = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, IT - 2, 0);  // two MFMAs (one when there are twelve)
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
  };

  const int nk = (g.K + CK - 1) / CK;
  const int nk4 = (nk + 3) & ~3;  // stages come in fours (the buffers are addressed statically)
  // Loads in flight, oldest first, whenever a wave reaches the barrier of
  // slab kt: [slab kt + 1] [slab kt + 2] [slab kt + 3]; the barrier needs the
  // first group, so two slabs' worth may stay outstanding.
  slab_load(sb0, 0, true);
  slab_load(sb0, 0, false);
  slab_load(sb1, 1, true);
  slab_load(sb1, 1, false);
  slab_load(sb2, 2, true);
  slab_load(sb2, 2, false);
  slab_load(sb3, 3, true);
  wait_loads_but<2 * NLOAD + IT>();  // everything but slab 0
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  if (CK > g.K) slab_clear_tail(sb0, 0);
  frags(0, sb0, 0);

  // The slab pipeline runs on across tiles: slabs nk4, nk4 + 1, .. of a tile are slabs 0, 1, ..
  // of the workgroup's next one (A and B are pointed at it just before the first such load), so
  // a tile's first slabs arrive while the previous tile finishes and is stored.  `last`: the
  // tile's last four stages.  `stores_between`: the wave has issued NSTORE stores since the loads
  // of the slab this stage waits for (vector memory operations retire in order and share the
  // counter), so that many more may be outstanding.
  auto stage = [&](int kt, auto b_c, auto fresh_c, bool last, bool stores_between) {
    constexpr int b = decltype(b_c)::value;  // kt & 3
    char* cur = buf(b);
    char* nxt = buf(b + 1);
    // first k-step (fragments already in set 0); meanwhile the second k-step's
    // fragments and the B half of slab kt + 3
    if (b == 1 && last) point_b(next_t);
    frags_and_loads(1, cur, 1, buf(b + 3), kt + 3 >= nk4 ? kt + 3 - nk4 : kt + 3, false);
    mfmas(0, fresh_c);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
    // This wave has read all it needs of slab kt; its share of slab kt + 1 has
    // landed once at most two slabs' worth of younger loads are outstanding.  Past the barrier
    // that holds for every wave: slab kt + 1 is complete, buffer b is free.
    if (stores_between) wait_loads_but<2 * NLOAD + NSTORE>();
    else wait_loads_but<2 * NLOAD>();  // two slabs' worth
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (kt + 1 < nk4 ? (kt + 2) * CK > g.K : CK > g.K) slab_clear_tail(nxt, kt + 1 < nk4 ? kt + 1 : 0);
    // second k-step; meanwhile the next slab's first fragments and the A half
    // of slab kt + 4 into the buffer just freed
    if (b == 0 && last) point_a(next_t);
    frags_and_loads(0, nxt, 0, cur, kt + 4 >= nk4 ? kt + 4 - nk4 : kt + 4, true);
    mfmas(1, std::false_type{});
    interleave();
    __builtin_amdgcn_sched_barrier(0);
  };

  // Epilogue of one tile, per wave and without a barrier: the wave stages 32 rows i x 64 columns j
  // of its quadrant at a time in its own corner of sOut and reads them back itself (a wave's
  // LDS operations execute in order), then writes 128-byte row segments.  It touches neither the
  // slab buffers nor the loads in flight into them.
  // Lane (l31, hh), register quad q of tile (jt, it): row i = 32 it + l31,
  // columns j = 32 jt + 8 q + 4 hh + 0..3.  Values are finished four at a time on their way from
  // the accumulators to LDS, so that few of them are live at once.
  bf16_t* sE = reinterpret_cast<bf16_t*>(sOut + wave * EPI_BYTES);
  auto store_tile = [&](const Tile& t) {
    bf16_t* C = reinterpret_cast<bf16_t*>(g.C) + (int64_t)t.bz * g.sC;
    // SwiGLU: accumulator tiles (0,1) and (2,3) give 32 output columns each, one pass per 32 rows;
    // otherwise two passes of 64 output columns
    constexpr int PASSES = MODE == BIG_SWIGLU ? 1 : 2;
    const int c8 = lane & 7, rsub = lane >> 3;  // 8 chunks of 8 output columns per row, 8 rows per instruction
    const uint32_t lane_off = (uint32_t)(rsub * g.ldc + c8 * 8) * 2u;
    const int col_end = MODE == BIG_SWIGLU ? g.N / 2 : MODE == BIG_PLAIN ? g.ldc : g.N;
    const __amdgpu_buffer_rsrc_t whole =
        __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(C), 0, MODE == BIG_COLUMN_OPS && g.regroup32 ? g.M * g.N * 2 : 0, RSRC_RAW);
    // Pass n = (it, p): 32 rows x 64 output columns.  convert: accumulators -> eight packed 8-byte
    // pieces per lane; write: those into the staging area; read_store: 16 bytes per lane back out
    // of it and to memory.  The passes are software-pipelined in the source (write n, convert
    // n + 1, read_store n): the conversions of the next pass fill the LDS round trip of this one.
    constexpr int NP = IT * PASSES;
    // The bias of the wave's 128 columns goes through LDS once per tile, requested before the
    // tile's first store: a load from memory issued between the stores would wait for them all
    // (vector memory operations retire in order).
    float* sBiasW = sColBias + (MODE == BIG_COLUMN_OPS ? wave * 128 : 0);
    if constexpr (MODE == BIG_COLUMN_OPS) {
      // the bias array only covers the segments that use it
      int first;
      const bool uses_bias = big_tile_bias_quad(g, t.n0 + wn + 4 * lane, &first) && lane < 32;
      f32x4 b4 = {0.f, 0.f, 0.f, 0.f};
      if (uses_bias) b4 = *reinterpret_cast<const f32x4*>(g.bias + first);
      if (lane < 32) *reinterpret_cast<f32x4*>(sBiasW + 4 * lane) = b4;
    }
    auto convert = [&](int n, u32x2* out) {
      const int it = n / PASSES, p = n % PASSES;
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const int jt = MODE == BIG_SWIGLU ? 2 * jj : 2 * p + jj;
        // column ops: a 32-column block never straddles segments (seg_len % 32 == 0)
        bool affine = false, sig = false;
        float alpha = 1.f;
        const int nb = t.n0 + wn + 32 * jt;
        if constexpr (MODE == BIG_COLUMN_OPS) {
          int op = SEG_BIAS_SCALE;
          sig = g.act_sigmoid != 0;
          if (g.epi == EPI_SEGMENTED) {
            op = (g.seg_ops >> (4 * (min(nb, g.N - 1) / g.seg_len))) & 15;
            sig = op == SEG_SIGMOID;
          }
          affine = op == SEG_BIAS_SCALE;
          if (affine) alpha = g.alpha;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float o[4];
          f32x4 bb = {0.f, 0.f, 0.f, 0.f};
          if constexpr (MODE == BIG_COLUMN_OPS) {
            if (affine && g.bias) bb = *reinterpret_cast<const f32x4*>(sBiasW + 32 * jt + 8 * q + 4 * hh);
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float v = acc_read(acc[jt][it][4 * q + e]);
            if constexpr (MODE == BIG_COLUMN_OPS) {
              v = (v + bb[e]) * alpha;
              if (sig) v = sigmoidf_(v);
            }
            if constexpr (MODE == BIG_SWIGLU) v = v * sigmoidf_(v) * acc_read(acc[jt + 1][it][4 * q + e]);
            o[e] = v;
          }
          out[4 * jj + q].x = pack2bf(o[0], o[1]);
          out[4 * jj + q].y = pack2bf(o[2], o[3]);
        }
      }
    };
    auto write = [&](const u32x2* in) {
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<u32x2*>(sE + l31 * LDE + 32 * jj + 8 * q + 4 * hh) = in[4 * jj + q];
    };
    // Bounds are enforced by the memory pipeline, not by branches (which would cut the
    // epilogue into many basic blocks): a buffer descriptor that ends with the last valid row
    // of this 32-row block drops rows past M, and lanes whose columns lie past the end
    // get an offset beyond any descriptor.  Every wave issues all its stores.
    auto read_store = [&](int n) {
      const int it = n / PASSES, p = n % PASSES;
      const int row0 = t.m0 + wm + 32 * it;
      const __amdgpu_buffer_rsrc_t rows32 = __builtin_amdgcn_make_buffer_rsrc(
          uniform_ptr(C + (int64_t)row0 * g.ldc), 0,
          __builtin_amdgcn_readfirstlane(max(0, min(32, g.M - row0)) * g.ldc * 2), RSRC_RAW);
      const int col0 = MODE == BIG_SWIGLU ? (t.n0 + wn) / 2 : t.n0 + wn + 64 * p;
      const uint32_t voff = c8 * 8 < col_end - col0 ? lane_off + (uint32_t)col0 * 2u : 0x80000000u;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int r = 8 * s + rsub;
        const u32x4 v = *reinterpret_cast<const u32x4*>(sE + r * LDE + c8 * 8);
        if (MODE == BIG_COLUMN_OPS && g.regroup32) {
          const int row = row0 + r, col = col0 + c8 * 8;
          const uint32_t off = ((((uint32_t)(row >> 5) * (uint32_t)(g.N >> 5) + (col >> 5)) * 32 + (row & 31)) * 32 + (col & 31)) * 2u;
          __builtin_amdgcn_raw_buffer_store_b128(v, whole, row < g.M && col < g.N ? off : 0x80000000u, 0, 0);
        } else {
          __builtin_amdgcn_raw_buffer_store_b128(v, rows32, voff + (uint32_t)(8 * s * g.ldc) * 2u, 0, 0);
        }
      }
    };
    u32x2 vals[2][8];
    convert(0, vals[0]);
#pragma unroll
    for (int n = 0; n < NP; ++n) {
      write(vals[n & 1]);
      if (n + 1 < NP) convert(n + 1, vals[(n + 1) & 1]);
      read_store(n);
    }
  };

  bool stored = false;  // a tile's epilogue (NSTORE stores per wave, whatever the bounds) lies behind
  while (true) {
    const bool has_next = tile_at(slot + slot_step, next_t);
    if (!has_next) next_t = cur_t;  // the loads past the tile's end then re-read its first slabs, unused
    // the tile's first four stages apart: its very first k-step starts the accumulators from the
    // constant zero (no 256 moves to clear them), and a branch on "first" inside the loop would
    // have the accumulators meet at its join
    stage(0, std::integral_constant<int, 0>{}, std::true_type{}, nk4 == 4, stored);
    stage(1, std::integral_constant<int, 1>{}, std::false_type{}, nk4 == 4, stored);
    stage(2, std::integral_constant<int, 2>{}, std::false_type{}, nk4 == 4, false);
    stage(3, std::integral_constant<int, 3>{}, std::false_type{}, nk4 == 4, false);
    for (int kt = 4; kt < nk4; kt += 4) {
      const bool last = kt + 4 == nk4;
      stage(kt, std::integral_constant<int, 0>{}, std::false_type{}, last, false);
      stage(kt + 1, std::integral_constant<int, 1>{}, std::false_type{}, last, false);
      stage(kt + 2, std::integral_constant<int, 2>{}, std::false_type{}, last, false);
      stage(kt + 3, std::integral_constant<int, 3>{}, std::false_type{}, last, false);
    }
    store_tile(cur_t);
    __builtin_amdgcn_sched_barrier(0);
    if (!has_next) break;
    stored = true;
    cur_t = next_t;
    slot += slot_step;
  }
  wait_loads_but<0>();  // nothing may be in flight into LDS when the workgroup ends
}

bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

// Layout assumptions the large tile shares over its modes.
static bool big_tile_layout_ok(const GemmArgs& g) {
  return !g.out_f32 && g.M > 0 && g.N > 0 && g.K > 0 && g.batch > 0 && (g.lda & 7) == 0 && (g.ldb & 7) == 0 &&
         (g.ldc & 7) == 0 && (g.K & 7) == 0 && g.K <= g.lda && g.K <= g.ldb && (g.sA & 7) == 0 && (g.sB & 7) == 0 &&
         (g.sC & 7) == 0 && al16(g.A) && al16(g.B) && al16(g.C) &&
         (int64_t)g.M * g.lda < (1ll << 30) && (int64_t)g.N * g.ldb < (1ll << 30) && g.ldc < (1 << 24);
}

// Plain bf16 batched NT product with the large tile; false if the operands do
// not meet its layout assumptions (the caller then takes the general GEMM).
bool contract_supported(const GemmArgs& g) {
  return g.epi == EPI_PLAIN && !g.bias && !g.act_sigmoid && g.alpha == 1.f && !g.regroup32 && !g.gate &&
         big_tile_layout_ok(g) && g.ldc >= ((g.N + 7) & ~7);
}

// Which large-tile instance can take this product with its epilogue: -1 = none.
int big_tile_mode(const GemmArgs& g) {
  if (!big_tile_layout_ok(g) || g.gate || g.res_f32 || g.res_bf16) return -1;
  if (g.epi == EPI_SWIGLU) return (g.N & 63) == 0 && g.ldc >= g.N / 2 && !g.regroup32 ? BIG_SWIGLU : -1;
  if (g.N & 7) return -1;
  if (!g.regroup32 && g.ldc < g.N) return -1;
  if (g.bias && !al16(g.bias)) return -1;
  if (g.epi == EPI_SEGMENTED) return g.seg_len > 0 && (g.seg_len & 31) == 0 && !g.regroup32 ? BIG_COLUMN_OPS : -1;
  if (g.epi != EPI_PLAIN) return -1;
  if (g.regroup32)
    return g.batch == 1 && (g.M & 31) == 0 && (g.N & 31) == 0 && (int64_t)g.M * g.N < (1ll << 30) ? BIG_COLUMN_OPS : -1;
  return (g.bias || g.act_sigmoid || g.alpha != 1.f) ? BIG_COLUMN_OPS : BIG_PLAIN;
}

void gemm_bias_span(const GemmArgs& g, bool big, int64_t* first, int64_t* last) {
  int64_t lo = INT64_MAX, hi = 0;
  if (g.bias && g.N > 0 && (g.epi != EPI_SEGMENTED || g.seg_len > 0)) {
    if (big) {
      // every (tile column, wave column, lane) of the epilogue's bias fetch
      for (int n0 = 0; n0 < g.N; n0 += CN)
        for (int wn = 0; wn < CN; wn += 128)
          for (int lane = 0; lane < 32; ++lane) {
            int f;
            if (!big_tile_bias_quad(g, n0 + wn + 4 * lane, &f)) continue;
            lo = std::min<int64_t>(lo, f);
            hi = std::max<int64_t>(hi, (int64_t)f + 4);
          }
    } else {
      // gemm_nt_kernel: chunk of up to 8 columns from every multiple of 8 below N
      for (int n = 0; n < g.N; n += 8) {
        if (!gemm_col_uses_bias(g, n)) continue;
        lo = std::min<int64_t>(lo, n);
        hi = std::max<int64_t>(hi, std::min<int64_t>(n + 8, g.N));
      }
    }
  }
  *first = hi > 0 ? lo : 0;
  *last = hi;
}

int launch_big_tile(const GemmArgs& g, int mode, hipStream_t stream) {
  if (!g.A || !g.B || !g.C) return AF3_ERR_BAD_ARG;
  if (mode != big_tile_mode(g) && !(mode == BIG_PLAIN && contract_supported(g))) return AF3_ERR_BAD_ARG;
  if (mode < BIG_PLAIN || mode > BIG_SWIGLU) return AF3_ERR_BAD_ARG;
  if (mode == BIG_COLUMN_OPS && g.bias) {
    // the epilogue fetches the bias in groups of four per lane: nothing it touches may lie outside the array
    int64_t first, last;
    gemm_bias_span(g, true, &first, &last);
    if (first < 0 || last > g.bias_len) return AF3_ERR_BAD_ARG;
  }
  const int64_t tiles_n = (g.N + CN - 1) / CN;
  const int64_t total4 = (int64_t)((g.M + 255) / 256) * tiles_n * g.batch;
  const int64_t total3 = (int64_t)((g.M + 191) / 192) * tiles_n * g.batch;
  // Rounds of workgroups on the device's CUs (one workgroup per CU) times the cost of one.  A 192 x 256
  // block costs 0.83 - 0.86 of a 256 x 256 one, not 0.75 (measured: pipeline fill and the epilogue do not
  // shrink with it), so it is taken for the plain product only when it saves more rounds than that:
  // N = 256 .. 576, not 768 (six rounds against five) or beyond.
  static int cus = 0;
  if (cus == 0) {
    int dev_id = 0;
    hipDeviceProp_t prop;
    cus = hipGetDevice(&dev_id) == hipSuccess && hipGetDeviceProperties(&prop, dev_id) == hipSuccess &&
                  prop.multiProcessorCount > 0
              ? prop.multiProcessorCount
              : 256;
  }
  const bool flat = ((total3 + cus - 1) / cus) * 7 < ((total4 + cus - 1) / cus) * 8;
  const int64_t total = flat ? total3 : total4;
  if (total > 0x3fffffff) return AF3_ERR_BAD_ARG;
  // persistent workgroups, one per CU (a multiple of 8: ids are dealt round-robin to the 8 XCDs)
  const int64_t blocks = std::min<int64_t>((total + 7) / 8 * 8, std::max(cus / 8 * 8, 8));
  const dim3 grid((unsigned)blocks), block(256);
  if (flat && mode == BIG_PLAIN) hipLaunchKernelGGL((contract_kernel<BIG_PLAIN, 3>), grid, block, 0, stream, g);
  else if (flat && mode == BIG_COLUMN_OPS) hipLaunchKernelGGL((contract_kernel<BIG_COLUMN_OPS, 3>), grid, block, 0, stream, g);
  else if (flat) hipLaunchKernelGGL((contract_kernel<BIG_SWIGLU, 3>), grid, block, 0, stream, g);
  else if (mode == BIG_PLAIN) hipLaunchKernelGGL(contract_kernel<BIG_PLAIN>, grid, block, 0, stream, g);
  else if (mode == BIG_COLUMN_OPS) hipLaunchKernelGGL(contract_kernel<BIG_COLUMN_OPS>, grid, block, 0, stream, g);
  else hipLaunchKernelGGL(contract_kernel<BIG_SWIGLU>, grid, block, 0, stream, g);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

int launch_contract(const GemmArgs& g, hipStream_t stream) {
  if (!g.A || !g.B || !g.C || !contract_supported(g)) return AF3_ERR_BAD_ARG;
  return launch_big_tile(g, BIG_PLAIN, stream);
}
