// Batched "NT" GEMM on bf16 MFMA:  C[b][m][n] = epi( sum_k A[b][m][k] * B[b][n][k] )
//
// Both operands are k-contiguous, which is the natural fragment order of
// v_mfma_f32_32x32x16_bf16, so a 16-byte load feeds one fragment.  The
// workgroup tile is 128x128 with a 64-deep k slab, double-buffered in LDS and
// prefetched through registers; four waves each own a 64x64 quadrant (2x2 MFMA
// tiles, 64 fp32 accumulators).
//
// This kernel carries the dense projections outside the 128-channel pair path
// (single / diffusion / atom attention and transitions) and the triangle
// contraction of small token counts; large products whose epilogue the
// 256x256-tile kernel (contract.hip) knows are handed to it by launch_gemm_nt.
#include <type_traits>

#include "common.h"
#include "kernels.h"

namespace {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDT = BK + 8;  // padded LDS row (bf16 elements): 144 B keeps 16-B reads conflict-free

constexpr int LDC_S = BN + 4;  // fp32 staging row stride of the C tile

// K_TAIL: K is not a multiple of the slab depth, so chunks past K have to be zeroed on their way to LDS.
template <bool OUT_F32, bool K_TAIL>
__global__ __launch_bounds__(256, 2) void gemm_nt_kernel(GemmArgs g) {
  // A/B slabs, double buffered; after the k loop the same memory stages the C tile
  __shared__ __attribute__((aligned(16))) bf16_t smem[2 * (BM + BN) * LDT];
  static_assert(BM * LDC_S * 4 <= 2 * (BM + BN) * LDT * 2, "C staging must fit");
  constexpr int STAGE = (BM + BN) * LDT;  // buffer `buf`: A slab at smem + buf * STAGE, B slab BM rows later
  float* sC = reinterpret_cast<float*>(smem);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;

  // XCD-aware mapping: workgroup ids are dealt round-robin to the 8 XCDs, so
  // id -> (xcd, slot) -> logical id makes each XCD walk a contiguous range of
  // (batch, n-tile, m-tile), m-tile fastest: the tiles that share a batch's A
  // and B panels run on one XCD and find them in its L2.
  const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
  const int total = tiles_m * tiles_n * g.batch;
  const int per_xcd = (total + 7) / 8;
  const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (logical >= total) return;
  const int tm = logical % tiles_m, tn = (logical / tiles_m) % tiles_n;
  const int bz = logical / (tiles_m * tiles_n);
  const int m0 = tm * BM, n0 = tn * BN;

  const bf16_t* A = g.A + (int64_t)bz * g.sA;
  const bf16_t* B = g.B + (int64_t)bz * g.sB;

  // each thread moves 4 16-byte chunks of A and 4 of B per k slab.  Two register
  // sets: a slab is requested two iterations before it goes to LDS.  The small
  // products this kernel is mostly used for (a few hundred rows, K = 384 ...
  // 1536) run on fewer workgroups than there are CUs, so each workgroup is one
  // chain of K / 64 memory round trips and nothing else covers their latency.
  const int ld_row = tid >> 3, ld_kc = (tid & 7) * 8;  // + 32 rows per step
  u32x4 ra[2][4], rb[2][4];
  const bf16_t* pa[4];
  const bf16_t* pb[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = ld_row + 32 * i;
    pa[i] = A + (int64_t)min(m0 + row, g.M - 1) * g.lda + ld_kc;
    pb[i] = B + (int64_t)min(n0 + row, g.N - 1) * g.ldb + ld_kc;
  }
  // unconditional loads (a chunk past K re-reads the row's first one) whose
  // values are zeroed on their way to LDS
  bool k_ok[2] = {true, true};
  auto gload = [&](int set, int k0) {
    k_ok[set] = k0 + ld_kc < g.K;
    const int kk = k_ok[set] ? k0 : -ld_kc;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ra[set][i] = *reinterpret_cast<const u32x4*>(pa[i] + kk);
      rb[set][i] = *reinterpret_cast<const u32x4*>(pb[i] + kk);
    }
  };
  auto sstore = [&](int set, int buf) {
    const u32x4 z = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = ld_row + 32 * i;
      *reinterpret_cast<u32x4*>(smem + buf * STAGE + row * LDT + ld_kc) = !K_TAIL || k_ok[set] ? ra[set][i] : z;
      *reinterpret_cast<u32x4*>(smem + buf * STAGE + (BM + row) * LDT + ld_kc) = !K_TAIL || k_ok[set] ? rb[set][i] : z;
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int nk = (g.K + BK - 1) / BK;
  gload(0, 0);
  gload(1, BK);  // past K when nk == 1: a clamped re-read, never stored
  sstore(0, 0);
  lds_barrier();

  // slab kt is in LDS buffer kt & 1, slab kt + 1 in register set (kt + 1) & 1,
  // and set kt & 1 (just stored) takes slab kt + 2
  auto stage = [&](int kt, auto par_c) {
    constexpr int par = decltype(par_c)::value;
    // Requested on every iteration, also past the last slab (a clamped
    // re-read that is never stored): a load under a condition leaves the
    // compiler unable to count the loads in flight, and it then waits for all
    // of them, the slab just requested included, before the LDS stores below.
    gload(par, (kt + 2) * BK);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = lds_frag(smem + par * STAGE, LDT, wm + 32 * i, ks * 16, lane);
#pragma unroll
      for (int j = 0; j < 2; ++j) fb[j] = lds_frag(smem + par * STAGE + BM * LDT, LDT, wn + 32 * j, ks * 16, lane);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mfma32(fa[i], fb[j], acc[i][j]);
    }
    // The next slab (requested one stage ago) goes into the other LDS buffer, which nobody reads during
    // this stage, while the matrix unit works: its eight stores are dealt out between the MFMAs of the
    // second half, behind the fragment reads (issued four ahead of the MFMAs that use them).  Unconditional,
    // so that it stays in one basic block with them: after the last slab it stores a clamped re-read that
    // nobody uses (the C tile is staged over it only after the barrier below).
    sstore(par ^ 1, par ^ 1);
    __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
    __builtin_amdgcn_sched_barrier(0);
    lds_barrier();
  };
  for (int kt = 0; kt < nk; kt += 2) {
    stage(kt, std::integral_constant<int, 0>{});
    if (kt + 1 < nk) stage(kt + 1, std::integral_constant<int, 1>{});
  }

  // ------------------------------------------------------------- epilogue
  // accumulators (lane = column, registers = rows) -> fp32 tile in LDS, then
  // each thread finishes 8 consecutive columns of a row with 16/32-byte stores
  const int cc = (tid & 15) * 8, r0 = tid >> 4;
  // Gate and residual of the thread's eight output chunks are requested here,
  // all at once and ahead of the staging: asked for one chunk at a time between
  // the stores (which may alias the residual, so the compiler keeps the order)
  // they would be eight memory round trips in a row at the end of a workgroup
  // that, in the small products, has nothing else to hide them behind.
  const bool gr_ahead = g.epi == EPI_GATE_RES && g.vec_ok && n0 + cc + 8 <= g.N && !g.res_f32 &&
                        (!g.gate || g.gate_per_row || g.gate_vec_ok) && (!g.res_bf16 || g.res_vec_ok);
  f32x4 gate_lo[8], gate_hi[8];
  u32x4 res_pk[8];
  float gate_row[8];
  if (gr_ahead) {
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int m = min(m0 + it * 16 + r0, g.M - 1), n = n0 + cc;
      gate_row[it] = 1.f;
      gate_lo[it] = gate_hi[it] = f32x4{1.f, 1.f, 1.f, 1.f};
      res_pk[it] = u32x4{0, 0, 0, 0};
      if (g.gate && g.gate_per_row) gate_row[it] = g.gate[m % g.gate_rows];
      else if (g.gate) {
        const float* gp = g.gate + (int64_t)(m % g.gate_rows) * g.ld_gate + n;
        gate_lo[it] = *reinterpret_cast<const f32x4*>(gp);
        gate_hi[it] = *reinterpret_cast<const f32x4*>(gp + 4);
      }
      if (g.res_bf16)
        res_pk[it] = *reinterpret_cast<const u32x4*>(g.res_bf16 + (int64_t)bz * g.sRes + (int64_t)m * g.ld_res + n);
    }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        sC[(wm + 32 * i + acc_row(r, lane)) * LDC_S + wn + 32 * j + (lane & 31)] = acc[i][j][r];
  lds_barrier();

  if (g.epi == EPI_SWIGLU) {
    // weight rows are packed in blocks of 64: 32 "a" rows then the 32 matching
    // "b" rows; output has N/2 columns.  Threads with cc < 64 produce 8 outputs each.
    if (cc >= 64) return;
    const int blk = cc >> 5, off = cc & 31;         // which 64-column block, offset inside its a half
    const int oc = n0 / 2 + cc;                     // first output column
    if (n0 + blk * 64 >= g.N) return;               // N % 64 == 0
    bf16_t* C = reinterpret_cast<bf16_t*>(g.C) + (int64_t)bz * g.sC;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int row = it * 16 + r0, m = m0 + row;
      if (m >= g.M) continue;
      const float* sa = sC + row * LDC_S + blk * 64 + off;
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) { const float a = sa[e], b = sa[32 + e]; o[e] = a * sigmoidf_(a) * b; }
      bf16_t* dst = C + (int64_t)m * g.ldc + oc;
      if (g.vec_ok) *reinterpret_cast<u32x4*>(dst) = pack8(o);
      else
#pragma unroll
        for (int e = 0; e < 8; ++e) dst[e] = f2bf(o[e]);
    }
    return;
  }

  const int n = n0 + cc;
  if (n >= g.N) return;
  const int nv = min(8, g.N - n);  // valid columns of this chunk
  float bias[8];
  int op = SEG_PLAIN;
#pragma unroll
  for (int e = 0; e < 8; ++e) bias[e] = 0.f;
  if (g.epi == EPI_SEGMENTED) {
    op = (g.seg_ops >> (4 * (n / g.seg_len))) & 15;  // seg_len % 8 == 0: a chunk never straddles segments
    if (gemm_col_uses_bias(g, n))
#pragma unroll
      for (int e = 0; e < 8; ++e) if (e < nv) bias[e] = g.bias[n + e];
  } else if (g.bias) {
#pragma unroll
    for (int e = 0; e < 8; ++e) if (e < nv) bias[e] = g.bias[n + e];
  }
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int row = it * 16 + r0, m = m0 + row;
    if (m >= g.M) continue;
    float v[8];
    const f32x4 lo = *reinterpret_cast<const f32x4*>(sC + row * LDC_S + cc);
    const f32x4 hi = *reinterpret_cast<const f32x4*>(sC + row * LDC_S + cc + 4);
    v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
    const bool full = g.vec_ok && nv == 8;
    if (g.epi == EPI_SEGMENTED) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (op == SEG_BIAS_SCALE) v[e] = (v[e] + bias[e]) * g.alpha;
        else if (op == SEG_SIGMOID) v[e] = sigmoidf_(v[e]);
      }
    } else if (gr_ahead) {
      const f32x4 gl = gate_lo[it], gh = gate_hi[it];
      const float gt[8] = {gl.x * gate_row[it], gl.y * gate_row[it], gl.z * gate_row[it], gl.w * gate_row[it],
                           gh.x * gate_row[it], gh.y * gate_row[it], gh.z * gate_row[it], gh.w * gate_row[it]};
      float rs[8];
      unpack8(res_pk[it], rs);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (v[e] + bias[e]) * gt[e] + rs[e];
    } else if (g.epi == EPI_GATE_RES) {
      const int64_t roff = (int64_t)bz * g.sRes + (int64_t)m * g.ld_res + n;
      float gt[8], rs[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) { gt[e] = 1.f; rs[e] = 0.f; }
      if (g.gate && g.gate_per_row) {
        const float f = g.gate[m % g.gate_rows];
#pragma unroll
        for (int e = 0; e < 8; ++e) gt[e] = f;
      } else if (g.gate) {
        const float* gp = g.gate + (int64_t)(m % g.gate_rows) * g.ld_gate + n;
#pragma unroll
        for (int e = 0; e < 8; ++e) if (e < nv) gt[e] = gp[e];
      }
      if (g.res_f32) {
#pragma unroll
        for (int e = 0; e < 8; ++e) if (e < nv) rs[e] = g.res_f32[roff + e];
      } else if (g.res_bf16) {
        if (full && g.res_vec_ok) unpack8(*reinterpret_cast<const u32x4*>(g.res_bf16 + roff), rs);
        else
#pragma unroll
          for (int e = 0; e < 8; ++e) if (e < nv) rs[e] = bf2f(g.res_bf16[roff + e]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (v[e] + bias[e]) * gt[e] + rs[e];
    } else {  // EPI_PLAIN
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        v[e] = (v[e] + bias[e]) * g.alpha;
        if (g.act_sigmoid) v[e] = sigmoidf_(v[e]);
      }
    }
    const int64_t off = g.regroup32
                            ? ((((int64_t)(m >> 5) * (g.N >> 5) + (n >> 5)) * 32 + (m & 31)) * 32 + (n & 31))
                            : (int64_t)bz * g.sC + (int64_t)m * g.ldc + n;
    if (OUT_F32) {
      float* dst = reinterpret_cast<float*>(g.C) + off;
      if (full) {
        *reinterpret_cast<f32x4*>(dst) = f32x4{v[0], v[1], v[2], v[3]};
        *reinterpret_cast<f32x4*>(dst + 4) = f32x4{v[4], v[5], v[6], v[7]};
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) if (e < nv) dst[e] = v[e];
      }
    } else {
      bf16_t* dst = reinterpret_cast<bf16_t*>(g.C) + off;
      if (full) *reinterpret_cast<u32x4*>(dst) = pack8(v);
      else
#pragma unroll
        for (int e = 0; e < 8; ++e) if (e < nv) dst[e] = f2bf(v[e]);
    }
  }
}

}  // namespace

// Products of at least 120 tiles of 256x256 go to the large-tile kernel where
// one of its epilogues fits: from there on the 128x128 tiles no longer fit
// the chip in one round (two workgroups per CU) and the large tile, with
// half the fragment reads per MFMA, is 1.3 to 1.45 times faster;
// below, the two kernels are within a few percent of each other and the
// small tile wins where it fills more CUs.
int gemm_big_tile_choice(const GemmArgs& g) {
  constexpr int64_t BIG_TILE_MIN_TILES = 120;
  const int64_t tiles = (int64_t)((g.M + 255) / 256) * ((g.N + 255) / 256) * g.batch;
  return g.M > 128 && g.N > 128 && tiles >= BIG_TILE_MIN_TILES ? big_tile_mode(g) : -1;
}

int launch_gemm_nt(const GemmArgs& g_in, hipStream_t stream) {
  GemmArgs g = g_in;
  if (g.M <= 0 || g.N <= 0 || g.K <= 0 || g.batch <= 0) return AF3_ERR_BAD_ARG;
  {
    const int big = gemm_big_tile_choice(g);
    if (big >= 0) return launch_big_tile(g, big, stream);
  }
  if ((g.K & 7) || (g.lda & 7) || (g.ldb & 7) || (g.sA & 7) || (g.sB & 7)) return AF3_ERR_BAD_ARG;
  if (((uintptr_t)g.A & 15) || ((uintptr_t)g.B & 15)) return AF3_ERR_BAD_ARG;
  if (g.epi == EPI_SWIGLU && ((g.N & 63) || g.out_f32)) return AF3_ERR_BAD_ARG;
  if (g.epi == EPI_SEGMENTED && (g.seg_len <= 0 || (g.seg_len & 7))) return AF3_ERR_BAD_ARG;
  if (g.gate && g.gate_rows <= 0) return AF3_ERR_BAD_ARG;
  if (g.bias) {
    int64_t first, last;
    gemm_bias_span(g, false, &first, &last);
    if (first < 0 || last > g.bias_len) return AF3_ERR_BAD_ARG;
  }
  if (g.regroup32 && (g.epi != EPI_PLAIN || g.batch != 1 || (g.M & 31) || (g.N & 31))) return AF3_ERR_BAD_ARG;
  // 16/32-byte stores need aligned rows; otherwise the epilogue stores element-wise
  const int esz = g.out_f32 ? 4 : 2;
  g.vec_ok = ((uintptr_t)g.C % 16 == 0) && ((g.ldc * esz) % 16 == 0) && ((g.sC * esz) % 16 == 0);
  g.gate_vec_ok = g.gate && !g.gate_per_row && ((uintptr_t)g.gate % 16 == 0) && (g.ld_gate % 4 == 0);
  g.res_vec_ok = g.res_bf16 && ((uintptr_t)g.res_bf16 % 16 == 0) && (g.ld_res % 8 == 0) && (g.sRes % 8 == 0);
  const int64_t total = (int64_t)((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN) * g.batch;
  const int64_t blocks = (total + 7) / 8 * 8;
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  dim3 grid((unsigned)blocks);
  const bool k_tail = (g.K % BK) != 0;
  if (g.out_f32 && k_tail) hipLaunchKernelGGL((gemm_nt_kernel<true, true>), grid, dim3(256), 0, stream, g);
  else if (g.out_f32) hipLaunchKernelGGL((gemm_nt_kernel<true, false>), grid, dim3(256), 0, stream, g);
  else if (k_tail) hipLaunchKernelGGL((gemm_nt_kernel<false, true>), grid, dim3(256), 0, stream, g);
  else hipLaunchKernelGGL((gemm_nt_kernel<false, false>), grid, dim3(256), 0, stream, g);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}
