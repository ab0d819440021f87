// fp32 check mode: plain, unfused fp32 kernels from which the host composes
// every operator of the hot path a second time, with fp32 storage and fp32 FMA
// arithmetic throughout.  They share no code with the bf16 MFMA kernels, so
// agreement between the two paths (and of this one with the CPU oracle to
// 1e-4) checks formulas, indexing, masks and weight packing independently of
// bf16 rounding.  Speed is not a goal here.
#include "common.h"
#include "kernels.h"

namespace {

// ---------------------------------------------------------------------------
// C[b][m][n] = epi( sum_k A[b][m*lda + k*ka] * B[b][n*ldb + k*kb] )
// generic strides (ka / kb let either operand be read transposed); 64x64 tile,
// 16-deep k slab in LDS, each thread a 4x4 patch.
// ---------------------------------------------------------------------------
constexpr int CT = 64, CK = 16;

__global__ __launch_bounds__(256) void ck_gemm_kernel(CkGemmArgs g) {
  __shared__ float sA[CK][CT + 1];
  __shared__ float sB[CK][CT + 1];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.x * CT, n0 = blockIdx.y * CT, bz = blockIdx.z;
  const float* A = g.A + (int64_t)bz * g.sA;
  const float* B = g.B + (int64_t)bz * g.sB;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < g.K; k0 += CK) {
    for (int idx = tid; idx < CT * CK; idx += 256) {
      const int r = idx / CK, k = idx % CK;
      const int m = m0 + r, n = n0 + r, kk = k0 + k;
      sA[k][r] = (m < g.M && kk < g.K) ? A[(int64_t)m * g.lda + (int64_t)kk * g.ka] : 0.f;
      sB[k][r] = (n < g.N && kk < g.K) ? B[(int64_t)n * g.ldb + (int64_t)kk * g.kb] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < CK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { a[i] = sA[k][ty * 4 + i]; b[i] = sB[k][tx * 4 + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= g.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= g.N) continue;
      float v = acc[i][j];
      if (g.bias) v += g.bias[n];
      v *= g.alpha;
      if (g.sigmoid) v = 1.0f / (1.0f + expf(-v));
      if (g.mul) v *= g.mul[(int64_t)(m % g.mul_rows) * g.ld_mul + n];
      if (g.add) v += g.add[(int64_t)bz * g.s_add + (int64_t)m * g.ld_add + n];
      g.C[(int64_t)bz * g.sC + (int64_t)m * g.ldc + n] = v;
    }
  }
}

// ---------------------------------------------------------------------------
// row LayerNorm in fp32 (one wave per row), optional affine / adaptive terms
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void ck_ln_kernel(CkNormArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.rows) return;
  const float* x = a.x + row * a.C;
  float s = 0.f;
  for (int c = lane; c < a.C; c += 64) s += x[c];
  const float mean = wave_sum(s) / (float)a.C;
  float q = 0.f;
  for (int c = lane; c < a.C; c += 64) { const float d = x[c] - mean; q += d * d; }
  const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)a.C + LN_EPS);
  const int64_t cr = a.cond_rows > 0 ? row % a.cond_rows : 0;
  float* y = a.y + row * a.C;
  for (int c = lane; c < a.C; c += 64) {
    float t = (x[c] - mean) * rstd;
    if (a.weight) t *= a.weight[c];
    if (a.bias) t += a.bias[c];
    if (a.scale) t = t / (1.0f + expf(-a.scale[cr * a.ld_cond + c])) + a.shift[cr * a.ld_cond + c];
    y[c] = t;
  }
}

// ---------------------------------------------------------------------------
// element-wise helpers
// ---------------------------------------------------------------------------
// triangle multiplication: v = proj * mask * sigmoid(gate); even channels -> a, odd -> b,
// written channel-major; incoming stores them transposed (a'[c][j][k] = a[k][j][c]).
__global__ void ck_trimul_split_kernel(const float* proj, const float* gate, const float* mask, float* a, float* b,
                                       int N, int C2, int incoming) {
  const int64_t total = (int64_t)N * N * C2;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
    const int ch2 = (int)(idx % C2);
    const int64_t pix = idx / C2;
    const int r = (int)(pix / N), c = (int)(pix % N);
    const float m = mask ? mask[pix] : 1.f;
    const float v = proj[idx] * m / (1.0f + expf(-gate[idx]));
    const int ch = ch2 >> 1;
    const int o = incoming ? c : r, k = incoming ? r : c;  // (outer, contraction) index
    float* dst = (ch2 & 1) ? b : a;
    dst[((int64_t)ch * N + o) * N + k] = v;
  }
}

// t[c][i][j] -> out[i][j][c]
__global__ void ck_chan_to_pix_kernel(const float* t, float* out, int N, int C) {
  const int64_t total = (int64_t)N * N * C;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(idx % C);
    const int64_t pix = idx / C;
    out[idx] = t[(int64_t)c * N * N + pix];
  }
}

// out[j][i][:] = in[i][j][:]
__global__ void ck_transpose_pix_kernel(const float* in, float* out, int N, int C) {
  const int64_t total = (int64_t)N * N * C;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(idx % C);
    const int64_t pix = idx / C;
    const int i = (int)(pix / N), j = (int)(pix % N);
    out[((int64_t)j * N + i) * C + c] = in[idx];
  }
}

// h[m][f] = silu(y[m][f]) * y[m][F + f]
__global__ void ck_swiglu_kernel(const float* y, float* h, int64_t M, int F) {
  const int64_t total = M * F;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t m = idx / F;
    const int f = (int)(idx % F);
    const float a = y[m * 2 * F + f], b = y[m * 2 * F + F + f];
    h[idx] = a / (1.0f + expf(-a)) * b;
  }
}

// y = x0 * x1 (flag 0) or x0 + x1 (flag 1)
__global__ void ck_binary_kernel(const float* x0, const float* x1, float* y, int64_t n, int add) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x)
    y[idx] = add ? x0[idx] + x1[idx] : x0[idx] * x1[idx];
}

// ---------------------------------------------------------------------------
// attention, one wave per (batch, head, query): two passes over the keys
// (max, then exp / sum / weighted values), everything fp32.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void ck_attention_kernel(CkAttnArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= (int64_t)a.B * a.H * a.Sq) return;
  const int q = (int)(w % a.Sq), h = (int)((w / a.Sq) % a.H), b = (int)(w / ((int64_t)a.Sq * a.H));
  const int bb = a.bias_mod > 0 ? b % a.bias_mod : b;
  const float* qp = a.q + (int64_t)b * a.q_sb + (int64_t)q * a.q_ss + h * a.d;
  const float* kb = a.k + (int64_t)b * a.k_sb + h * a.d;
  const float* vb = a.v + (int64_t)b * a.v_sb + h * a.d;
  float qv[64];
  for (int c = 0; c < a.d; ++c) qv[c] = qp[c];
  const bool qpad = a.qpad ? a.qpad[(int64_t)bb * a.Sq + q] == 0.f : false;
  auto logit = [&](int k) {
    const float* kp = kb + (int64_t)k * a.k_ss;
    float s = 0.f;
    for (int c = 0; c < a.d; ++c) s = fmaf(qv[c], kp[c], s);
    if (a.bias) s += a.bias[(int64_t)bb * a.bias_sb + (int64_t)h * a.bias_sh + (int64_t)q * a.bias_sq + (int64_t)k * a.bias_sk];
    if (a.key_mask && a.key_mask[(int64_t)b * a.km_sb + k] == 0.f) s = -1e9f;
    if (qpad && a.kpad[(int64_t)bb * a.Sk + k] == 0.f) s += 1e9f;
    return s;
  };
  float mx = -__builtin_huge_valf();
  for (int k = lane; k < a.Sk; k += 64) mx = fmaxf(mx, logit(k));
  mx = wave_max(mx);
  float l = 0.f, o[64];
  for (int c = 0; c < a.d; ++c) o[c] = 0.f;
  for (int k = lane; k < a.Sk; k += 64) {
    const float p = expf(logit(k) - mx);
    l += p;
    const float* vp = vb + (int64_t)k * a.v_ss;
    for (int c = 0; c < a.d; ++c) o[c] = fmaf(p, vp[c], o[c]);
  }
  l = wave_sum(l);
  float* op = a.out + (int64_t)b * a.o_sb + (int64_t)q * a.o_ss + h * a.d;
  for (int c = 0; c < a.d; ++c) {
    const float t = wave_sum(o[c]);
    if (lane == 0) op[c] = t / l;
  }
}

unsigned grid_for(int64_t total) {
  const int64_t b = (total + 255) / 256, cap = 65535 * 16;
  return (unsigned)(b < cap ? b : cap);
}

}  // namespace

int launch_ck_gemm(const CkGemmArgs& g, hipStream_t s) {
  if (!g.A || !g.B || !g.C || g.M <= 0 || g.N <= 0 || g.K <= 0 || g.batch <= 0 || g.batch > 65535) return AF3_ERR_BAD_ARG;
  if (g.mul && g.mul_rows <= 0) return AF3_ERR_BAD_ARG;
  const int64_t gy = (g.N + CT - 1) / CT;
  if (gy > 65535) return AF3_ERR_BAD_ARG;
  dim3 grid((unsigned)((g.M + CT - 1) / CT), (unsigned)gy, (unsigned)g.batch);
  hipLaunchKernelGGL(ck_gemm_kernel, grid, dim3(256), 0, s, g);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}
int launch_ck_norm(const CkNormArgs& a, hipStream_t s) {
  if (!a.x || !a.y || a.rows <= 0 || a.C <= 0) return AF3_ERR_BAD_ARG;
  if ((a.scale == nullptr) != (a.shift == nullptr) || (a.scale && a.cond_rows <= 0)) return AF3_ERR_BAD_ARG;
  hipLaunchKernelGGL(ck_ln_kernel, dim3((unsigned)((a.rows + 3) / 4)), dim3(256), 0, s, a);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}
int launch_ck_elementwise(int op, const float* x0, const float* x1, const float* x2, float* y0, float* y1,
                          int64_t n0, int64_t n1, int flag, hipStream_t s) {
  if (!x0 || !y0 || n0 <= 0) return AF3_ERR_BAD_ARG;
  switch (op) {
    case CK_TRIMUL_SPLIT:
      if (!x1 || !y1 || n0 > 8192) return AF3_ERR_BAD_ARG;
      // n1: pair channels (0 = 128); proj / gate hold twice as many
      if (n1 < 0 || n1 > 4096) return AF3_ERR_BAD_ARG;
      hipLaunchKernelGGL(ck_trimul_split_kernel, dim3(grid_for(n0 * n0 * 2 * (n1 ? n1 : 128))), dim3(256), 0, s, x0, x1, x2,
                         y0, y1, (int)n0, (int)(2 * (n1 ? n1 : 128)), flag);
      break;
    case CK_CHAN_TO_PIX:
      if (n0 > 8192 || n1 <= 0) return AF3_ERR_BAD_ARG;
      hipLaunchKernelGGL(ck_chan_to_pix_kernel, dim3(grid_for(n0 * n0 * n1)), dim3(256), 0, s, x0, y0, (int)n0, (int)n1);
      break;
    case CK_TRANSPOSE_PIX:
      if (n0 > 8192 || n1 <= 0) return AF3_ERR_BAD_ARG;
      hipLaunchKernelGGL(ck_transpose_pix_kernel, dim3(grid_for(n0 * n0 * n1)), dim3(256), 0, s, x0, y0, (int)n0, (int)n1);
      break;
    case CK_SWIGLU:
      if (n1 <= 0) return AF3_ERR_BAD_ARG;
      hipLaunchKernelGGL(ck_swiglu_kernel, dim3(grid_for(n0 * n1)), dim3(256), 0, s, x0, y0, n0, (int)n1);
      break;
    case CK_BINARY:
      if (!x1) return AF3_ERR_BAD_ARG;
      hipLaunchKernelGGL(ck_binary_kernel, dim3(grid_for(n0)), dim3(256), 0, s, x0, x1, y0, n0, flag);
      break;
    default:
      return AF3_ERR_BAD_ARG;
  }
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}
int launch_ck_attention(const CkAttnArgs& a, hipStream_t s) {
  if (!a.q || !a.k || !a.v || !a.out || a.B <= 0 || a.H <= 0 || a.Sq <= 0 || a.Sk <= 0 || a.d <= 0 || a.d > 64)
    return AF3_ERR_BAD_ARG;
  if ((a.qpad == nullptr) != (a.kpad == nullptr)) return AF3_ERR_BAD_ARG;
  const int64_t waves = (int64_t)a.B * a.H * a.Sq;
  const int64_t blocks = (waves + 3) / 4;
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  hipLaunchKernelGGL(ck_attention_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}
