// Batched "NT" GEMM on bf16 MFMA:  C[b][m][n] = epi( sum_k A[b][m][k] * B[b][n][k] )
//
// Both operands are k-contiguous, which is the natural fragment order of
// v_mfma_f32_32x32x16_bf16, so a 16-byte load feeds one fragment.  The
// workgroup tile is 128x128 with a 64-deep k slab, double-buffered in LDS and
// prefetched through registers; four waves each own a 64x64 quadrant (2x2 MFMA
// tiles, 64 fp32 accumulators).
//
// This kernel carries the triangle-multiplication contraction (batch = 128
// channels, M = N = K = N_token) and every dense projection outside the
// 128-channel pair path (single / diffusion / atom attention and transitions).
#include "common.h"
#include "kernels.h"

namespace {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDT = BK + 8;  // padded LDS row (bf16 elements): 144 B keeps 16-B reads conflict-free

template <bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_nt_kernel(GemmArgs g) {
  __shared__ __attribute__((aligned(16))) bf16_t sA[2][BM * LDT];
  __shared__ __attribute__((aligned(16))) bf16_t sB[2][BN * LDT];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;

  // blockIdx.x walks m-tiles fastest: workgroups in flight together work on
  // the same batch (channel) and few B panels, which keeps them in L2/MALL.
  const int tiles_m = (g.M + BM - 1) / BM;
  const int tm = blockIdx.x % tiles_m, tn = blockIdx.x / tiles_m;
  const int bz = blockIdx.y;
  const int m0 = tm * BM, n0 = tn * BN;

  const bf16_t* A = g.A + (int64_t)bz * g.sA;
  const bf16_t* B = g.B + (int64_t)bz * g.sB;

  // each thread moves 4 16-byte chunks of A and 4 of B per k slab
  const int ld_row = tid >> 3, ld_kc = (tid & 7) * 8;  // + 32 rows per step
  u32x4 ra[4], rb[4];

  auto gload = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = ld_row + 32 * i;
      const int k = k0 + ld_kc;
      const int am = min(m0 + row, g.M - 1), bn = min(n0 + row, g.N - 1);
      const u32x4 z = {0, 0, 0, 0};
      ra[i] = (k < g.K) ? *reinterpret_cast<const u32x4*>(A + (int64_t)am * g.lda + k) : z;
      rb[i] = (k < g.K) ? *reinterpret_cast<const u32x4*>(B + (int64_t)bn * g.ldb + k) : z;
    }
  };
  auto sstore = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = ld_row + 32 * i;
      *reinterpret_cast<u32x4*>(&sA[buf][row * LDT + ld_kc]) = ra[i];
      *reinterpret_cast<u32x4*>(&sB[buf][row * LDT + ld_kc]) = rb[i];
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
  gload(0);
  sstore(0);
  lds_barrier();

  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) gload((kt + 1) * BK);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = lds_frag(sA[buf], LDT, wm + 32 * i, ks * 16, lane);
#pragma unroll
      for (int j = 0; j < 2; ++j) fb[j] = lds_frag(sB[buf], LDT, wn + 32 * j, ks * 16, lane);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mfma32(fa[i], fb[j], acc[i][j]);
    }
    if (kt + 1 < nk) sstore(buf ^ 1);
    lds_barrier();
  }

  // ---------------------------------------------------------------- epilogue
  const int col_l = lane & 31;
  if (g.epi == EPI_SWIGLU) {
    // weight rows are packed in blocks of 64: 32 "a" rows then the 32 matching
    // "b" rows, so MFMA tile j=0 holds a and j=1 holds b for the same hidden
    // units; output has N/2 columns.
    bf16_t* C = reinterpret_cast<bf16_t*>(g.C) + (int64_t)bz * g.sC;
    const int oc = (n0 + wn) / 2 + col_l;
    if (n0 + wn < g.N) {  // N % 64 == 0: a 64-column wave span is all in or all out
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + wm + 32 * i + acc_row(r, lane);
          if (m < g.M) {
            const float a = acc[i][0][r], b = acc[i][1][r];
            C[(int64_t)m * g.ldc + oc] = f2bf(a * sigmoidf_(a) * b);
          }
        }
    }
    return;
  }

#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int n = n0 + wn + 32 * j + col_l;
    if (n >= g.N) continue;
    float bias = 0.f;
    int op = SEG_PLAIN;
    if (g.epi == EPI_SEGMENTED) {
      const int seg = n / g.seg_len;
      op = (g.seg_ops >> (4 * seg)) & 15;
      if (op == SEG_BIAS_SCALE && g.bias) bias = g.bias[n];
    } else if (g.bias) {
      bias = g.bias[n];
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm + 32 * i + acc_row(r, lane);
        if (m >= g.M) continue;
        float v = acc[i][j][r];
        if (g.epi == EPI_SEGMENTED) {
          if (op == SEG_BIAS_SCALE) v = (v + bias) * g.alpha;
          else if (op == SEG_SIGMOID) v = sigmoidf_(v);
        } else if (g.epi == EPI_GATE_RES) {
          v += bias;
          if (g.gate) v *= g.gate[(int64_t)(m % g.gate_rows) * g.ld_gate + n];
          if (g.res_f32) v += g.res_f32[(int64_t)bz * g.sRes + (int64_t)m * g.ld_res + n];
          if (g.res_bf16) v += bf2f(g.res_bf16[(int64_t)bz * g.sRes + (int64_t)m * g.ld_res + n]);
        } else {  // EPI_PLAIN
          v = (v + bias) * g.alpha;
          if (g.act_sigmoid) v = sigmoidf_(v);
        }
        const int64_t off = (int64_t)bz * g.sC + (int64_t)m * g.ldc + n;
        if (OUT_F32) reinterpret_cast<float*>(g.C)[off] = v;
        else reinterpret_cast<bf16_t*>(g.C)[off] = f2bf(v);
      }
  }
}

}  // namespace

int launch_gemm_nt(const GemmArgs& g, hipStream_t stream) {
  if (g.M <= 0 || g.N <= 0 || g.K <= 0 || g.batch <= 0) return AF3_ERR_BAD_ARG;
  if ((g.K & 7) || (g.lda & 7) || (g.ldb & 7) || (g.sA & 7) || (g.sB & 7)) return AF3_ERR_BAD_ARG;
  if (((uintptr_t)g.A & 15) || ((uintptr_t)g.B & 15)) return AF3_ERR_BAD_ARG;
  if (g.epi == EPI_SWIGLU && ((g.N & 63) || g.out_f32)) return AF3_ERR_BAD_ARG;
  if (g.epi == EPI_SEGMENTED && g.seg_len <= 0) return AF3_ERR_BAD_ARG;
  if (g.gate && g.gate_rows <= 0) return AF3_ERR_BAD_ARG;
  const int tiles = ((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN);
  dim3 grid(tiles, g.batch);
  if (g.out_f32) hipLaunchKernelGGL(gemm_nt_kernel<true>, grid, dim3(256), 0, stream, g);
  else hipLaunchKernelGGL(gemm_nt_kernel<false>, grid, dim3(256), 0, stream, g);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}
