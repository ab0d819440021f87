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
// What paces the kernel is the CU's vector memory path: it accepts 64 bytes
// per cycle, so the 32 KB of operands that go with 32 MFMAs per wave (1024
// cycles of the matrix unit) occupy it for 512 cycles, and a wave that issues
// a load into a full queue stalls with its MFMAs behind it.  A lone wave per
// SIMD has nobody to cover for it.  So:
//   * slabs (32 k deep) go from global memory straight into LDS
//     (global_load_lds_dwordx4: no staging registers, no LDS stores in the
//     instruction stream);
//   * the loads are spread evenly, one per four MFMAs per wave, which keeps the
//     memory path half busy all the time instead of saturated in bursts;
//   * four LDS buffers: a load is issued two to three slabs (2000-3000 cycles)
//     before anybody waits for it, about the latency of a miss that goes to HBM;
//   * the one barrier per slab sits between its two k-steps, after the wave has
//     read all its fragments of the slab: the MFMAs of the second k-step cover
//     the barrier and the first fragment reads of the next slab, and the
//     buffer is free for refill the moment the barrier is passed.
// A load puts lane l's 16 bytes at LDS base + 16 l, so rows cannot be padded;
// instead the four 16-byte chunks of a 64-byte row are permuted, chunk c of row
// r living at position c ^ ((r >> 2) & 3), which makes the fragment reads (32
// rows x one chunk per half-wave) conflict-free over the 64 banks.  The
// permutation is applied on the global side, where a lane is free to fetch
// any chunk.
//
// The accumulators hold T^T tiles (B fragments as the MFMA's A operand), so a
// lane owns one output row i and four consecutive columns j per register quad:
// the epilogue packs those to 8 bytes, stages each wave's quadrant through LDS
// and writes full 256-byte rows.
#include <type_traits>

#include "common.h"
#include "kernels.h"

namespace {

// The block is 64 IT x 256: IT = 4 MFMA tiles per wave along i (256 x 256), or IT = 3 (192 x 256) where
// that saves enough rounds of workgroups (N = 384: tiles of 256 would be half empty).
constexpr int CN = 256, CK = 32;
constexpr int ROWB = CK * 2;            // bytes of a slab row in LDS (unpadded)
constexpr int SLAB = (256 + CN) * ROWB;  // 32 KB at IT = 4: A rows first, then B rows
constexpr int LDE = 128 + 8;            // LDS row stride of a wave's staged output quadrant (bf16)
constexpr int EPI_BYTES = 128 * LDE * 2;  // one wave's output quadrant
constexpr int BUF_BYTES = SLAB > EPI_BYTES ? SLAB : EPI_BYTES;
constexpr int NBUF = 4;

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// 64 lanes x 16 bytes from global (uniform base + per-lane byte offset) to
// 1 KB of LDS starting at the wave-uniform address dst
__device__ __forceinline__ void load_to_lds(const char* base, uint32_t off, char* dst) {
  __builtin_amdgcn_global_load_lds((gptr_t)(base + off), (lptr_t)dst, 16, 0, 0);
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
  // Four arrays, not one: the compiler then knows that a load in flight to one
  // buffer cannot alias a fragment read from another and does not make the
  // read wait for it.
  __shared__ __attribute__((aligned(1024))) char sb0[BUF_BYTES];
  __shared__ __attribute__((aligned(1024))) char sb1[BUF_BYTES];
  __shared__ __attribute__((aligned(1024))) char sb2[BUF_BYTES];
  __shared__ __attribute__((aligned(1024))) char sb3[BUF_BYTES];
  auto buf = [&](int i) -> char* { return (i & 3) == 0 ? sb0 : (i & 3) == 1 ? sb1 : (i & 3) == 2 ? sb2 : sb3; };

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hh = lane >> 5, l31 = lane & 31;
  const int wm = (wave >> 1) * WM, wn = (wave & 1) * 128;

  // XCD-aware mapping: workgroup ids are dealt round-robin to the 8 XCDs, so
  // id -> (xcd, slot) -> logical id makes each XCD walk a contiguous range of
  // (channel, j-tile, i-tile), i-tile fastest: the tiles that share a channel's
  // A and B panels run on one XCD and find them in its L2.
  const int tiles_m = (g.M + CM - 1) / CM, tiles_n = (g.N + CN - 1) / CN;
  const int total = tiles_m * tiles_n * g.batch;
  const int per_xcd = (total + 7) / 8;
  const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (logical >= total) return;
  int tm = logical % tiles_m, tn = (logical / tiles_m) % tiles_n;
  const int bz = logical / (tiles_m * tiles_n);
  if (g.batch == 1 && (tiles_m & 3) == 0 && (tiles_n & 1) == 0) {
    // One large product: an XCD that walks whole columns of tiles re-reads all of
    // A for every column, and A (8 MB at 4096 x 1024) does not stay in its 4 MB
    // L2.  Deal the XCDs a 4 x 2 grid of rectangles instead: a quarter of A stays
    // resident while the XCD streams through its half of B once.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int mq = tiles_m >> 2, nh = tiles_n >> 1;
    tm = (xcd & 3) * mq + slot % mq;
    tn = (xcd >> 2) * nh + slot / mq;
  }
  const int m0 = tm * CM, n0 = tn * CN;

  const char* A = reinterpret_cast<const char*>(g.A + (int64_t)bz * g.sA);
  const char* B = reinterpret_cast<const char*>(g.B + (int64_t)bz * g.sB);

  // Per slab a wave issues IT loads for A and four for B: load i covers rows
  // 16 IT wave + 16 i .. + 16 of A, 64 wave + 16 i .. + 16 of B (one 64-byte row per 4 lanes).  The lane at position
  // pc of row r fetches chunk pc ^ ((r >> 2) & 3) = pc ^ (lane >> 4).  Rows past
  // the end repeat the last one (what they produce lands in output rows that
  // are never stored or in columns N..ldc-1 of T, which no consumer reads); a
  // chunk past K is fetched from the row's first slab instead and zeroed in
  // LDS before the slab is used.
  const int ld_r = lane >> 2;
  const int ld_c = (lane & 3) ^ (lane >> 4);
  uint32_t offa[4], offb[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int rowa = 16 * IT * wave + 16 * i + ld_r, rowb = 64 * wave + 16 * i + ld_r;
    offa[i] = ((uint32_t)min(m0 + rowa, g.M - 1) * (uint32_t)g.lda + ld_c * 8) * 2u;
    offb[i] = ((uint32_t)min(n0 + rowb, g.N - 1) * (uint32_t)g.ldb + ld_c * 8) * 2u;
  }
  // Half a slab: `first` = the wave's loads of A, else its four of B.
  // kt may run past the last slab (such loads re-read slab 0 and are never used).
  auto slab_load = [&](char* dst, int kt, bool first) {
    const int k0 = kt * CK;
    const uint32_t kb = k0 + ld_c * 8 < g.K ? (uint32_t)k0 * 2u : 0u;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (first) {
        if (i < IT) load_to_lds(A, offa[i] + kb, dst + (16 * IT * wave + 16 * i) * ROWB);
      } else {
        load_to_lds(B, offb[i] + kb, dst + SLAB_A + (64 * wave + 16 * i) * ROWB);
      }
    }
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
#pragma unroll
  for (int jt = 0; jt < 4; ++jt)
#pragma unroll
    for (int it = 0; it < IT; ++it)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[jt][it][r] = 0.f;

  bf16x8 fa[2][IT], fb[2][4];  // set 0: first k-step of a slab, set 1: second
  auto frags = [&](int set, const char* b, int ks) {
#pragma unroll
    for (int it = 0; it < IT; ++it)
      fa[set][it] = as_frag(*reinterpret_cast<const u32x4*>(b + a_base + it * (32 * ROWB) + fo[ks]));
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
      fb[set][jt] = as_frag(*reinterpret_cast<const u32x4*>(b + b_base + jt * (32 * ROWB) + fo[ks]));
  };
  auto mfmas = [&](int set) {
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
#pragma unroll
      for (int it = 0; it < IT; ++it) acc[jt][it] = mfma32(fb[set][jt], fa[set][it], acc[jt][it]);
  };
  // 4 IT MFMAs with IT + 4 fragment reads and up to 4 loads between them
  auto interleave = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, IT - 2, 0);  // two MFMAs (one when there are twelve)
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one global load
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

  auto stage = [&](int kt, auto b_c) {
    constexpr int b = decltype(b_c)::value;  // kt & 3
    char* cur = buf(b);
    char* nxt = buf(b + 1);
    // first k-step (fragments already in set 0); meanwhile the second k-step's
    // fragments and the B half of slab kt + 3
    frags(1, cur, 1);
    slab_load(buf(b + 3), kt + 3, false);
    mfmas(0);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
    // This wave has read all it needs of slab kt; its share of slab kt + 1 has
    // landed once at most two slabs' worth of younger loads are outstanding.  Past the barrier
    // that holds for every wave: slab kt + 1 is complete, buffer b is free.
    wait_loads_but<2 * NLOAD>();  // two slabs' worth
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if ((kt + 2) * CK > g.K && kt + 1 < nk4) slab_clear_tail(nxt, kt + 1);
    // second k-step; meanwhile the next slab's first fragments and the A half
    // of slab kt + 4 into the buffer just freed
    frags(0, nxt, 0);
    slab_load(cur, kt + 4, true);
    mfmas(1);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
  };
  for (int kt = 0; kt < nk4; kt += 4) {
    stage(kt, std::integral_constant<int, 0>{});
    stage(kt + 1, std::integral_constant<int, 1>{});
    stage(kt + 2, std::integral_constant<int, 2>{});
    stage(kt + 3, std::integral_constant<int, 3>{});
  }

  // ------------------------------------------------------------- epilogue
  // Drain the loads that ran ahead (they target the buffers about to be
  // reused) and let every wave finish its fragment reads.  Then a wave stages
  // its own (32 IT)x128 quadrant (rows i, columns j) in buffer `wave` and reads it
  // back itself (a wave's LDS operations execute in order): no further barrier.
  // Lane (l31, hh), register quad q of tile (jt, it): row i = 32 it + l31,
  // columns j = 32 jt + 8 q + 4 hh + 0..3.
  wait_loads_but<0>();
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  bf16_t* sE = reinterpret_cast<bf16_t*>(buf(wave));
  // Values are finished four at a time on their way from the accumulators to
  // LDS, so that few of them are live at once.
  constexpr int JSTEP = MODE == BIG_SWIGLU ? 2 : 1;  // SwiGLU: tiles (0,1) and (2,3) give 32 output columns each
#pragma unroll
  for (int jt = 0; jt < 4; jt += JSTEP) {
    // column ops: a 32-column block never straddles segments (seg_len % 32 == 0)
    bool affine = false, sig = false;
    float alpha = 1.f;
    const int nb = n0 + wn + 32 * jt;
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
      float bb[4] = {0.f, 0.f, 0.f, 0.f};
      if constexpr (MODE == BIG_COLUMN_OPS) {
        if (affine && g.bias) {
          const f32x4 b = *reinterpret_cast<const f32x4*>(g.bias + min(nb + 8 * q + 4 * hh, g.N - 4));
          bb[0] = b.x; bb[1] = b.y; bb[2] = b.z; bb[3] = b.w;
        }
      }
#pragma unroll
      for (int it = 0; it < IT; ++it) {
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float v = acc[jt][it][4 * q + e];
          if constexpr (MODE == BIG_COLUMN_OPS) {
            v = (v + bb[e]) * alpha;
            if (sig) v = sigmoidf_(v);
          }
          if constexpr (MODE == BIG_SWIGLU) v = v * sigmoidf_(v) * acc[jt + 1][it][4 * q + e];
          o[e] = v;
        }
        u32x2 v2;
        v2.x = pack2bf(o[0], o[1]);
        v2.y = pack2bf(o[2], o[3]);
        *reinterpret_cast<u32x2*>(sE + (32 * it + l31) * LDE + 32 * (jt / JSTEP) + 8 * q + 4 * hh) = v2;
      }
    }
  }
  bf16_t* C = reinterpret_cast<bf16_t*>(g.C) + (int64_t)bz * g.sC;
  if constexpr (MODE == BIG_SWIGLU) {
    const int c8 = lane & 7, rsub = lane >> 3;  // 8 chunks of 8 output columns per row, 8 rows per instruction
    const int col = (n0 + wn) / 2 + c8 * 8;
#pragma unroll
    for (int s = 0; s < 4 * IT; ++s) {
      const int r = 8 * s + rsub;
      const int row = m0 + wm + r;
      const u32x4 v = *reinterpret_cast<const u32x4*>(sE + r * LDE + c8 * 8);
      if (row < g.M && col < g.N / 2) *reinterpret_cast<u32x4*>(C + (int64_t)row * g.ldc + col) = v;
    }
  } else {
    const int c16 = lane & 15, rsub = lane >> 4;  // 16 chunks of 8 columns per row, 4 rows per instruction
    const int col = n0 + wn + c16 * 8;
    const int col_end = MODE == BIG_PLAIN ? g.ldc : g.N;
#pragma unroll
    for (int s = 0; s < 8 * IT; ++s) {
      const int r = 4 * s + rsub;
      const int row = m0 + wm + r;
      const u32x4 v = *reinterpret_cast<const u32x4*>(sE + r * LDE + c16 * 8);
      if (row < g.M && col < col_end) {
        int64_t off = (int64_t)row * g.ldc + col;
        if (MODE == BIG_COLUMN_OPS && g.regroup32)
          off = (((int64_t)(row >> 5) * (g.N >> 5) + (col >> 5)) * 32 + (row & 31)) * 32 + (col & 31);
        *reinterpret_cast<u32x4*>(C + off) = v;
      }
    }
  }
}

bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

// Layout assumptions the large tile shares over its modes.
static bool big_tile_layout_ok(const GemmArgs& g) {
  return !g.out_f32 && g.M > 0 && g.N > 0 && g.K > 0 && g.batch > 0 && (g.lda & 7) == 0 && (g.ldb & 7) == 0 &&
         (g.ldc & 7) == 0 && (g.K & 7) == 0 && g.K <= g.lda && g.K <= g.ldb && (g.sA & 7) == 0 && (g.sB & 7) == 0 &&
         (g.sC & 7) == 0 && al16(g.A) && al16(g.B) && al16(g.C) &&
         (int64_t)g.M * g.lda < (1ll << 30) && (int64_t)g.N * g.ldb < (1ll << 30);
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
  if (g.regroup32) return g.batch == 1 && (g.M & 31) == 0 && (g.N & 31) == 0 ? BIG_COLUMN_OPS : -1;
  return (g.bias || g.act_sigmoid || g.alpha != 1.f) ? BIG_COLUMN_OPS : BIG_PLAIN;
}

int launch_big_tile(const GemmArgs& g, int mode, hipStream_t stream) {
  if (!g.A || !g.B || !g.C) return AF3_ERR_BAD_ARG;
  if (mode != big_tile_mode(g) && !(mode == BIG_PLAIN && contract_supported(g))) return AF3_ERR_BAD_ARG;
  if (mode < BIG_PLAIN || mode > BIG_SWIGLU) return AF3_ERR_BAD_ARG;
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
  const bool flat = mode == BIG_PLAIN && ((total3 + cus - 1) / cus) * 7 < ((total4 + cus - 1) / cus) * 8;
  const int64_t total = flat ? total3 : total4;
  const int64_t blocks = (total + 7) / 8 * 8;
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  const dim3 grid((unsigned)blocks), block(256);
  if (flat) hipLaunchKernelGGL((contract_kernel<BIG_PLAIN, 3>), grid, block, 0, stream, g);
  else if (mode == BIG_PLAIN) hipLaunchKernelGGL(contract_kernel<BIG_PLAIN>, grid, block, 0, stream, g);
  else if (mode == BIG_COLUMN_OPS) hipLaunchKernelGGL(contract_kernel<BIG_COLUMN_OPS>, grid, block, 0, stream, g);
  else hipLaunchKernelGGL(contract_kernel<BIG_SWIGLU>, grid, block, 0, stream, g);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

int launch_contract(const GemmArgs& g, hipStream_t stream) {
  if (!g.A || !g.B || !g.C || !contract_supported(g)) return AF3_ERR_BAD_ARG;
  return launch_big_tile(g, BIG_PLAIN, stream);
}
