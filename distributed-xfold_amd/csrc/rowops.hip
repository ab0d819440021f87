// Row-wise LayerNorm / adaptive LayerNorm for the single, diffusion and atom
// activations (any channel count that is a multiple of 8).  One wave owns one
// row: 16-byte loads, two-pass statistics in registers, a 64-lane reduction,
// bf16 output ready to be an MFMA operand.  HBM-bound.
#include "common.h"
#include "kernels.h"

namespace {

constexpr int MAX_CHUNKS = 4;  // 64 lanes * 8 channels * 4 = 2048 channels at most

template <typename TIn>
__global__ __launch_bounds__(256) void ln_rows_kernel(RowNormArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.rows) return;
  const TIn* x = reinterpret_cast<const TIn*>(a.x) + row * a.ldx;
  float v[MAX_CHUNKS][8];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < MAX_CHUNKS; ++i) {
    const int c = (i * 64 + lane) * 8;
    if (c < a.C) {
      Elem<TIn>::load8(x + c, v[i]);
#pragma unroll
      for (int e = 0; e < 8; ++e) s += v[i][e];
    }
  }
  const float mean = wave_sum(s) / (float)a.C;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < MAX_CHUNKS; ++i) {
    const int c = (i * 64 + lane) * 8;
    if (c < a.C) {
#pragma unroll
      for (int e = 0; e < 8; ++e) { const float d = v[i][e] - mean; q += d * d; }
    }
  }
  const float rstd = rsqrtf(wave_sum(q) / (float)a.C + LN_EPS);
  const int64_t crow = a.cond_rows > 0 ? row % a.cond_rows : 0;
  bf16_t* y = a.y + row * a.ldy;
#pragma unroll
  for (int i = 0; i < MAX_CHUNKS; ++i) {
    const int c = (i * 64 + lane) * 8;
    if (c < a.C) {
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float t = (v[i][e] - mean) * rstd;
        if (a.weight) t *= a.weight[c + e];
        if (a.bias) t += a.bias[c + e];
        if (a.scale) t = sigmoidf_(a.scale[crow * a.ld_cond + c + e]) * t + a.shift[crow * a.ld_cond + c + e];
        o[e] = t;
      }
      *reinterpret_cast<u32x4*>(y + c) = pack8(o);
    }
  }
}

}  // namespace

int launch_row_norm(const RowNormArgs& a, hipStream_t stream) {
  if (a.rows <= 0 || a.C <= 0 || (a.C & 7) || a.C > 64 * 8 * MAX_CHUNKS) return AF3_ERR_BAD_ARG;
  if ((a.ldx & 7) || (a.ldy & 7) || ((uintptr_t)a.x & 15) || ((uintptr_t)a.y & 15)) return AF3_ERR_BAD_ARG;
  if ((a.scale == nullptr) != (a.shift == nullptr)) return AF3_ERR_BAD_ARG;
  if (a.scale && a.cond_rows <= 0) return AF3_ERR_BAD_ARG;
  const unsigned blocks = (unsigned)((a.rows + 3) / 4);
  if (a.x_f32) hipLaunchKernelGGL(ln_rows_kernel<float>, dim3(blocks), dim3(256), 0, stream, a);
  else hipLaunchKernelGGL(ln_rows_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, a);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}
