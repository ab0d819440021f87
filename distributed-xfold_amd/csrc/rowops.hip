// Row-wise LayerNorm / adaptive LayerNorm for the single, diffusion and atom
// activations (any channel count that is a multiple of 8).  One wave owns one
// row (or, for narrow rows, a group of 1..16 lanes does): 16-byte loads,
// two-pass statistics in registers, a shuffle reduction, bf16 output ready to
// be an MFMA operand.  HBM-bound.
#include <type_traits>

#include "common.h"
#include "kernels.h"

namespace {

constexpr int MAX_CHUNKS = 4;  // 64 lanes * 8 channels * 4 = 2048 channels at most

// Eight consecutive fp32 parameters (the channel offset is a multiple of 8):
// two 16-byte loads when the launcher found the array aligned for them.
__device__ __forceinline__ void load8f(const float* p, bool vec, float* out) {
  if (vec) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p);
    const f32x4 b = *reinterpret_cast<const f32x4*>(p + 4);
    out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
    out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = p[e];
  }
}

// y = LN(x) [* weight] [+ bias], then [sigmoid(scale) * y + shift], 8 channels
__device__ __forceinline__ void finish8(const RowNormArgs& a, const float* v, float mean, float rstd, int c,
                                        int64_t crow, float* o) {
  float w[8], b[8], sc[8], sh[8];
  if (a.weight) load8f(a.weight + c, a.param_vec, w);
  if (a.bias) load8f(a.bias + c, a.param_vec, b);
  if (a.scale) {
    load8f(a.scale + crow * a.ld_cond + c, a.cond_vec, sc);
    load8f(a.shift + crow * a.ld_cond + c, a.cond_vec, sh);
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float t = (v[e] - mean) * rstd;
    if (a.weight) t *= w[e];
    if (a.bias) t += b[e];
    if (a.scale) t = sigmoidf_(sc[e]) * t + sh[e];
    o[e] = t;
  }
}

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
      finish8(a, v[i], mean, rstd, c, crow, o);
      *reinterpret_cast<u32x4*>(y + c) = pack8(o);
    }
  }
}

// Narrow rows (C <= 128, e.g. the 16-channel atom pair conditioning with its
// millions of rows): G lanes per row, 64 / G rows per wave, so a wave still
// moves a full kilobyte per instruction instead of one lane group's worth.
template <typename TIn, int G>
__global__ __launch_bounds__(256) void ln_rows_small_kernel(RowNormArgs a) {
  constexpr int RPW = 64 / G;
  const int lane = threadIdx.x & 63, sub = lane % G;
  const int64_t row = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * RPW + lane / G;
  const bool ok = row < a.rows && sub * 8 < a.C;
  const int64_t rr = row < a.rows ? row : a.rows - 1;
  const int c = sub * 8 < a.C ? sub * 8 : 0;
  float v[8];
  Elem<TIn>::load8(reinterpret_cast<const TIn*>(a.x) + rr * a.ldx + c, v);
  float s = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) { v[e] = ok ? v[e] : 0.f; s += v[e]; }
#pragma unroll
  for (int m = 1; m < G; m <<= 1) s += __shfl_xor(s, m);
  const float mean = s / (float)a.C;
  float q = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) { const float d = ok ? v[e] - mean : 0.f; q += d * d; }
#pragma unroll
  for (int m = 1; m < G; m <<= 1) q += __shfl_xor(q, m);
  const float rstd = rsqrtf(q / (float)a.C + LN_EPS);
  if (!ok) return;
  const int64_t crow = a.cond_rows > 0 ? row % a.cond_rows : 0;
  float o[8];
  finish8(a, v, mean, rstd, c, crow, o);
  *reinterpret_cast<u32x4*>(a.y + row * a.ldy + c) = pack8(o);
}

template <typename TIn>
int launch_small(const RowNormArgs& a, hipStream_t stream) {
  const int chunks = a.C / 8;
  const int g = chunks <= 1 ? 1 : chunks <= 2 ? 2 : chunks <= 4 ? 4 : chunks <= 8 ? 8 : 16;
  const int64_t rows_per_block = 4 * (64 / g);
  const int64_t blocks = (a.rows + rows_per_block - 1) / rows_per_block;
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  const dim3 grid((unsigned)blocks), block(256);
  switch (g) {
    case 1: hipLaunchKernelGGL((ln_rows_small_kernel<TIn, 1>), grid, block, 0, stream, a); break;
    case 2: hipLaunchKernelGGL((ln_rows_small_kernel<TIn, 2>), grid, block, 0, stream, a); break;
    case 4: hipLaunchKernelGGL((ln_rows_small_kernel<TIn, 4>), grid, block, 0, stream, a); break;
    case 8: hipLaunchKernelGGL((ln_rows_small_kernel<TIn, 8>), grid, block, 0, stream, a); break;
    default: hipLaunchKernelGGL((ln_rows_small_kernel<TIn, 16>), grid, block, 0, stream, a); break;
  }
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

}  // namespace

int launch_row_norm(const RowNormArgs& a_in, hipStream_t stream) {
  RowNormArgs a = a_in;
  auto al16 = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  a.param_vec = al16(a.weight) && al16(a.bias);
  a.cond_vec = al16(a.scale) && al16(a.shift) && (a.ld_cond & 3) == 0;
  if (a.rows <= 0 || a.C <= 0 || (a.C & 7) || a.C > 64 * 8 * MAX_CHUNKS) return AF3_ERR_BAD_ARG;
  if ((a.ldx & 7) || (a.ldy & 7) || ((uintptr_t)a.x & 15) || ((uintptr_t)a.y & 15)) return AF3_ERR_BAD_ARG;
  if ((a.scale == nullptr) != (a.shift == nullptr)) return AF3_ERR_BAD_ARG;
  if (a.scale && a.cond_rows <= 0) return AF3_ERR_BAD_ARG;
  if (a.C <= 128) return a.x_f32 ? launch_small<float>(a, stream) : launch_small<bf16_t>(a, stream);
  const unsigned blocks = (unsigned)((a.rows + 3) / 4);
  if (a.x_f32) hipLaunchKernelGGL(ln_rows_kernel<float>, dim3(blocks), dim3(256), 0, stream, a);
  else hipLaunchKernelGGL(ln_rows_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, a);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

// ------------------------------------------------------------------ transpose
// out[c][r] = in[r][c] for a bf16 matrix, 64 x 64 tiles through LDS: 16-byte
// loads along the input rows, 16-byte stores along the output rows.  (The dense
// kernels want the summation index innermost in both operands; the MSA
// operators sum over MSA rows or tokens, which the activations carry as outer
// indices.)
namespace {
constexpr int TT = 64, TLD = TT + 2;  // 33 dwords per row: the column reads of a wave spread over the banks

__global__ __launch_bounds__(256) void transpose_kernel(const bf16_t* in, bf16_t* out, int64_t rows, int64_t cols) {
  __shared__ bf16_t tile[TT * TLD];
  const int tid = threadIdx.x;
  const int64_t tiles_c = (cols + TT - 1) / TT;
  const int64_t r0 = (blockIdx.x / tiles_c) * TT, c0 = (blockIdx.x % tiles_c) * TT;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int idx = tid + 256 * i, r = idx >> 3, ch = (idx & 7) * 8;
    u32x4 v = {0, 0, 0, 0};
    if (r0 + r < rows && c0 + ch < cols) v = *reinterpret_cast<const u32x4*>(in + (r0 + r) * cols + c0 + ch);
    uint32_t* dst = reinterpret_cast<uint32_t*>(&tile[r * TLD + ch]);  // rows are 4-byte aligned only
    dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int idx = tid + 256 * i, c = idx >> 3, rh = (idx & 7) * 8;
    if (c0 + c >= cols || r0 + rh >= rows) continue;
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      w[e] = (uint32_t)tile[(rh + 2 * e) * TLD + c] | ((uint32_t)tile[(rh + 2 * e + 1) * TLD + c] << 16);
    *reinterpret_cast<u32x4*>(out + (c0 + c) * rows + r0 + rh) = u32x4{w[0], w[1], w[2], w[3]};
  }
}
// out[b][t][c] = (sum over slots a with idx[t][a] >= 0 of relu(src[b][idx[t][a]][c])) / count[t].
// One thread per (b, t, 8 channels): the rows of all slots are requested
// before any is used.
template <int SLOTS_MAX>
__global__ __launch_bounds__(256) void gathered_relu_mean_kernel(const bf16_t* __restrict__ src,
                                                                  const int* __restrict__ idx,
                                                                  const float* __restrict__ count,
                                                                  float* __restrict__ out, int64_t batch,
                                                                  int64_t n_src, int64_t n_out, int slots, int C) {
  const int cch = C >> 3;
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= batch * n_out * cch) return;
  const int c8 = (int)(item % cch);
  const int64_t t = (item / cch) % n_out, b = item / ((int64_t)cch * n_out);
  const int* rows = idx + t * slots;
  const bf16_t* base = src + b * n_src * C + c8 * 8;
  u32x4 v[SLOTS_MAX];
  bool live[SLOTS_MAX];
#pragma unroll
  for (int a = 0; a < SLOTS_MAX; ++a) {
    const int r = a < slots ? rows[a] : -1;
    live[a] = r >= 0;
    v[a] = *reinterpret_cast<const u32x4*>(base + (int64_t)(r >= 0 ? r : 0) * C);
  }
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
#pragma unroll
  for (int a = 0; a < SLOTS_MAX; ++a) {
    float f[8];
    unpack8(v[a], f);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += live[a] ? fmaxf(f[e], 0.f) : 0.f;
  }
  const float d = count[t];
  float* dst = out + (b * n_out + t) * C + c8 * 8;
  *reinterpret_cast<f32x4*>(dst) = f32x4{acc[0] / d, acc[1] / d, acc[2] / d, acc[3] / d};
  *reinterpret_cast<f32x4*>(dst + 4) = f32x4{acc[4] / d, acc[5] / d, acc[6] / d, acc[7] / d};
}

// out[b][q][c] = cond[q][c] + sum_k pos[b][rows[q]][k] * w[c][k]  (rows[q] < 0: no position term)
// One thread per (b, q, 8 channels).
template <typename TOUT>
__global__ __launch_bounds__(256) void atom_position_features_kernel(const float* __restrict__ pos,
                                                                      const int* __restrict__ rows,
                                                                      const float* __restrict__ w,
                                                                      const float* __restrict__ cond,
                                                                      TOUT* __restrict__ out, int64_t batch,
                                                                      int64_t n_slots, int64_t n_q, int C) {
  const int cch = C >> 3;
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= batch * n_q * cch) return;
  const int c0 = (int)(item % cch) * 8;
  const int64_t q = (item / cch) % n_q, b = item / ((int64_t)cch * n_q);
  const int r = rows[q];
  const float* pp = pos + (b * n_slots + (r >= 0 ? r : 0)) * 3;
  const float live = r >= 0 ? 1.f : 0.f;
  const float x = pp[0] * live, y = pp[1] * live, z = pp[2] * live;
  const float* cp = cond + q * C + c0;
  const f32x4 ca = *reinterpret_cast<const f32x4*>(cp), cb = *reinterpret_cast<const f32x4*>(cp + 4);
  const float cv[8] = {ca.x, ca.y, ca.z, ca.w, cb.x, cb.y, cb.z, cb.w};
  float o[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float* we = w + (c0 + e) * 3;
    // the order of the eager steps: ((x w0 + y w1) + z w2), then + cond
    o[e] = ((x * we[0] + y * we[1]) + z * we[2]) + cv[e];
  }
  TOUT* dst = out + (b * n_q + q) * C + c0;
  if constexpr (std::is_same<TOUT, float>::value) {
    *reinterpret_cast<f32x4*>(dst) = f32x4{o[0], o[1], o[2], o[3]};
    *reinterpret_cast<f32x4*>(dst + 4) = f32x4{o[4], o[5], o[6], o[7]};
  } else {
    *reinterpret_cast<u32x4*>(dst) = pack8(o);
  }
}

// out[b][q][:] = bf16((rows[q] >= 0 ? src[b][rows[q]][:] : 0) + add[b][q][:]), one thread per 8 channels
__global__ __launch_bounds__(256) void gather_rows_add_kernel(const bf16_t* __restrict__ src,
                                                               const int* __restrict__ rows,
                                                               const bf16_t* __restrict__ add, bf16_t* __restrict__ out,
                                                               int64_t batch, int64_t n_src, int64_t n_q, int C) {
  const int cch = C >> 3;
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= batch * n_q * cch) return;
  const int c0 = (int)(item % cch) * 8;
  const int64_t q = (item / cch) % n_q, b = item / ((int64_t)cch * n_q);
  const int r = rows[q];
  const u32x4 sv = *reinterpret_cast<const u32x4*>(src + (b * n_src + (r >= 0 ? r : 0)) * C + c0);
  const u32x4 av = *reinterpret_cast<const u32x4*>(add + (b * n_q + q) * C + c0);
  float f[8], g[8];
  unpack8(sv, f);
  unpack8(av, g);
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = (r >= 0 ? f[e] : 0.f) + g[e];
  *reinterpret_cast<u32x4*>(out + (b * n_q + q) * C + c0) = pack8(f);
}

// out[b][t][k] = rows[t] >= 0 ? sum_c bf16(LayerNorm(x[b][rows[t]])[c] * ln_w[c]) * w[k][c] : 0   (k < 3, C = 128)
// One thread per output position: its row is 256 contiguous bytes.
__global__ __launch_bounds__(256) void ln_project3_gather_kernel(const bf16_t* __restrict__ x,
                                                                  const int* __restrict__ rows,
                                                                  const float* __restrict__ ln_w,
                                                                  const float* __restrict__ w, float* __restrict__ out,
                                                                  int64_t batch, int64_t n_src, int64_t n_out) {
  constexpr int C = 128;
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= batch * n_out) return;
  const int64_t t = item % n_out, b = item / n_out;
  const int r = rows[t];
  float* dst = out + item * 3;
  if (r < 0) {
    dst[0] = dst[1] = dst[2] = 0.f;
    return;
  }
  const bf16_t* row = x + (b * n_src + r) * C;
  float v[C];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < C / 8; ++i) {
    unpack8(*reinterpret_cast<const u32x4*>(row + 8 * i), v + 8 * i);
#pragma unroll
    for (int e = 0; e < 8; ++e) s += v[8 * i + e];
  }
  const float mean = s / (float)C;
  float q = 0.f;
#pragma unroll
  for (int c = 0; c < C; ++c) { const float d = v[c] - mean; q += d * d; }
  const float rstd = rsqrtf(q / (float)C + LN_EPS);
  float o0 = 0.f, o1 = 0.f, o2 = 0.f;
#pragma unroll
  for (int c = 0; c < C; ++c) {
    const float y = bf2f(f2bf((v[c] - mean) * rstd * ln_w[c]));  // the normalised row is a bf16 tensor in the eager steps
    o0 += y * w[c];
    o1 += y * w[C + c];
    o2 += y * w[2 * C + c];
  }
  dst[0] = o0; dst[1] = o1; dst[2] = o2;
}

// ----------------------------------------------------------------------------
// softmax over the rows of a [rows][cols] fp32 array with an additive key mask -> bf16.
// One wave per row, three passes over the row (it stays in the caches): maximum, sum of
// exponentials, normalised values.  y[r][k] = softmax_k(x[r][k] + 1e9 (mask[k] - 1)),
// columns cols .. ldy - 1 of y are zero.
// ----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void softmax_rows_kernel(const float* __restrict__ x, const float* __restrict__ mask,
                                                          bf16_t* __restrict__ y, int64_t rows, int cols, int64_t ldy) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const float* xr = x + r * cols;
  auto logit = [&](int k) { return xr[k] + (mask ? 1e9f * (mask[k] - 1.f) : 0.f); };
  float m = -__builtin_huge_valf();
  for (int k = lane; k < cols; k += 64) m = fmaxf(m, logit(k));
  m = wave_max(m);
  float s = 0.f;
  for (int k = lane; k < cols; k += 64) s += __expf(logit(k) - m);
  s = wave_sum(s);
  const float inv = 1.f / s;
  bf16_t* yr = y + r * ldy;
  for (int k = lane; k < ldy; k += 64) yr[k] = k < cols ? f2bf(__expf(logit(k) - m) * inv) : (bf16_t)0;
}

// ----------------------------------------------------------------------------
// Narrow fp32 layers of the atom conditioning: y[r][:] = (res ? res[r][:] : 0) + W f(x[r][:]),
// f = relu or the identity, W [NOUT][k] with NOUT = 16 or 3 outputs and k a multiple of 4 up to
// 128.  One thread per row, the weights in LDS, plain fp32 FMAs (these layers set up per-batch
// conditioning in fp32; they are far too narrow for the matrix units).
// ----------------------------------------------------------------------------
template <int NOUT>
__global__ __launch_bounds__(256) void narrow_linear_f32_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                               const float* __restrict__ res, float* __restrict__ y,
                                                               int64_t rows, int k, int relu_in) {
  __shared__ __attribute__((aligned(16))) float sW[NOUT * 128];
  for (int i = threadIdx.x; i < NOUT * k; i += 256) sW[i] = w[i];
  __syncthreads();
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= rows) return;
  float acc[NOUT];
#pragma unroll
  for (int o = 0; o < NOUT; ++o) acc[o] = res ? res[r * NOUT + o] : 0.f;
  const float* xr = x + r * k;
  for (int c = 0; c < k; c += 4) {
    f32x4 v = *reinterpret_cast<const f32x4*>(xr + c);
    if (relu_in) { v.x = fmaxf(v.x, 0.f); v.y = fmaxf(v.y, 0.f); v.z = fmaxf(v.z, 0.f); v.w = fmaxf(v.w, 0.f); }
#pragma unroll
    for (int o = 0; o < NOUT; ++o) {
      const f32x4 ww = *reinterpret_cast<const f32x4*>(sW + o * k + c);
      acc[o] = fmaf(v.x, ww.x, fmaf(v.y, ww.y, fmaf(v.z, ww.z, fmaf(v.w, ww.w, acc[o]))));
    }
  }
#pragma unroll
  for (int o = 0; o < NOUT; ++o) y[r * NOUT + o] = acc[o];
}


// ----------------------------------------------------------------------------
// Pair logits of the windowed atom transformer: per row of 16 conditioning channels a LayerNorm (weight, no
// bias) and a 16 -> n_out projection, n_out = blocks x heads, each output written to its own
// [block][subset][head][query][key] plane: the layout the attention kernel reads its bias in.  Rows are
// (subset, query, key) in this order, `group` = queries x keys rows per subset.  One thread per row, fp32.
// ----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void atom_pair_logits_kernel(const float* __restrict__ x, const float* __restrict__ ln_w,
                                                               const float* __restrict__ w, float* __restrict__ out,
                                                               int64_t rows, int64_t group, int64_t n_groups, int n_blocks,
                                                               int n_head) {
  __shared__ __attribute__((aligned(16))) float sW[32 * 16];
  const int n_out = n_blocks * n_head;
  // the LayerNorm weight goes into the projection: (xhat * g) . w = xhat . (g * w)
  for (int i = threadIdx.x; i < n_out * 16; i += 256) sW[i] = w[i] * ln_w[i & 15];
  __syncthreads();
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= rows) return;
  float v[16];
#pragma unroll
  for (int c = 0; c < 16; c += 4) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(x + r * 16 + c);
    v[c] = t.x; v[c + 1] = t.y; v[c + 2] = t.z; v[c + 3] = t.w;
  }
  float mean = 0.f;
#pragma unroll
  for (int c = 0; c < 16; ++c) mean += v[c];
  mean *= 1.f / 16;
  float var = 0.f;
#pragma unroll
  for (int c = 0; c < 16; ++c) { v[c] -= mean; var = fmaf(v[c], v[c], var); }
  const float rstd = rsqrtf(var * (1.f / 16) + LN_EPS);
  const int64_t s = r / group, qk = r - s * group;
  for (int o = 0; o < n_out; ++o) {
    float acc = 0.f;
#pragma unroll
    for (int c = 0; c < 16; c += 4) {
      const f32x4 ww = *reinterpret_cast<const f32x4*>(sW + o * 16 + c);
      acc = fmaf(v[c], ww.x, fmaf(v[c + 1], ww.y, fmaf(v[c + 2], ww.z, fmaf(v[c + 3], ww.w, acc))));
    }
    const int blk = o / n_head, h = o - blk * n_head;
    out[(((int64_t)blk * n_groups + s) * n_head + h) * group + qk] = acc * rstd;
  }
}


// ----------------------------------------------------------------------------
// Pair conditioning of the windowed atom attention, one pass per (subset, query, key):
//   a = row[s,q] + col[s,k] + [both atoms exist] tp[token(s,q), token(s,k)]
//       + valid * (W_off (pos_q - pos_k) + W_dist / (1 + |pos_q - pos_k|^2)) + valid * w_valid,
//   valid = the two atoms share a reference frame (uid_q == uid_k),
//   out = a + W3 relu(W2 relu(W1 relu(a)))                      (16 channels, fp32 throughout).
// One thread per (s, q, k), the weights in LDS.  Every term used to be a pass of its own over the
// [S, Q, K, 16] tensor.
// ----------------------------------------------------------------------------
struct AtomPairCondArgs {
  const float *row, *col;           // [S*Q][16], [S*K][16]
  const float* tp;                  // [n_tok*n_tok][16] or null
  const int *tq, *tk;               // token of query atom (s,q) / key atom (s,k), negative: no atom
  const float *q_pos, *k_pos;       // [S*Q][3], [S*K][3]
  const int *q_uid, *k_uid;
  const float *w_off, *w_dist, *w_valid, *w1, *w2, *w3;  // [16][3], [16], [16], [16][16] x 3
  float* out;
  int64_t S;
  int Q, K, n_tok;
};

__global__ __launch_bounds__(256) void atom_pair_cond_kernel(AtomPairCondArgs a) {
  __shared__ __attribute__((aligned(16))) float sW[3 * 256 + 16 * 4 + 16 + 16];
  float* sOff = sW + 768;   // [16][4]: w_off rows padded to four
  float* sDist = sOff + 64;
  float* sValid = sDist + 16;
  for (int i = threadIdx.x; i < 768; i += 256) sW[i] = (i < 256 ? a.w1 : i < 512 ? a.w2 : a.w3)[i & 255];
  if (threadIdx.x < 64) sOff[threadIdx.x] = (threadIdx.x & 3) < 3 ? a.w_off[(threadIdx.x >> 2) * 3 + (threadIdx.x & 3)] : 0.f;
  if (threadIdx.x < 16) { sDist[threadIdx.x] = a.w_dist[threadIdx.x]; sValid[threadIdx.x] = a.w_valid[threadIdx.x]; }
  __syncthreads();
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= a.S * a.Q * a.K) return;
  const int k = (int)(r % a.K);
  const int64_t sq = r / a.K, sk = (sq / a.Q) * a.K + k;
  float v[16];
#pragma unroll
  for (int c = 0; c < 16; c += 4) {
    const f32x4 x = *reinterpret_cast<const f32x4*>(a.row + sq * 16 + c), y = *reinterpret_cast<const f32x4*>(a.col + sk * 16 + c);
    v[c] = x.x + y.x; v[c + 1] = x.y + y.y; v[c + 2] = x.z + y.z; v[c + 3] = x.w + y.w;
  }
  if (a.tp) {
    const int tq = a.tq[sq], tk = a.tk[sk];
    if (tq >= 0 && tk >= 0) {
      const float* t = a.tp + ((int64_t)tq * a.n_tok + tk) * 16;
#pragma unroll
      for (int c = 0; c < 16; c += 4) {
        const f32x4 x = *reinterpret_cast<const f32x4*>(t + c);
        v[c] += x.x; v[c + 1] += x.y; v[c + 2] += x.z; v[c + 3] += x.w;
      }
    }
  }
  if (a.q_uid[sq] == a.k_uid[sk]) {
    const float dx = a.q_pos[sq * 3] - a.k_pos[sk * 3], dy = a.q_pos[sq * 3 + 1] - a.k_pos[sk * 3 + 1],
                dz = a.q_pos[sq * 3 + 2] - a.k_pos[sk * 3 + 2];
    const float inv = 1.0f / (1.0f + (dx * dx + dy * dy + dz * dz));
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      const f32x4 w = *reinterpret_cast<const f32x4*>(sOff + 4 * c);
      v[c] += fmaf(dz, w.z, fmaf(dy, w.y, dx * w.x)) + inv * sDist[c] + sValid[c];
    }
  }
  // three 16 x 16 layers with a relu on the way in; the residual is the unactivated a
  auto layer = [&](const float* w, const float* in, float* out) {
#pragma unroll
    for (int o = 0; o < 16; ++o) {
      float acc = 0.f;
#pragma unroll
      for (int c = 0; c < 16; c += 4) {
        const f32x4 ww = *reinterpret_cast<const f32x4*>(w + o * 16 + c);
        acc = fmaf(fmaxf(in[c], 0.f), ww.x, fmaf(fmaxf(in[c + 1], 0.f), ww.y,
                   fmaf(fmaxf(in[c + 2], 0.f), ww.z, fmaf(fmaxf(in[c + 3], 0.f), ww.w, acc))));
      }
      out[o] = acc;
    }
  };
  float h1[16], h2[16];
  layer(sW, v, h1);
  layer(sW + 256, h1, h2);
  layer(sW + 512, h2, h1);
#pragma unroll
  for (int c = 0; c < 16; c += 4) {
    const f32x4 o = {v[c] + h1[c], v[c + 1] + h1[c + 1], v[c + 2] + h1[c + 2], v[c + 3] + h1[c + 3]};
    *reinterpret_cast<f32x4*>(a.out + r * 16 + c) = o;
  }
}

}  // namespace

int launch_gather_rows_add(const bf16_t* src, const int* rows, const bf16_t* add, bf16_t* out, int64_t batch,
                           int64_t n_src, int64_t n_q, int channels, hipStream_t stream) {
  if (!src || !rows || !add || !out || batch <= 0 || n_src <= 0 || n_q <= 0 || channels <= 0 || (channels & 7))
    return AF3_ERR_BAD_ARG;
  if (((uintptr_t)src & 15) || ((uintptr_t)add & 15) || ((uintptr_t)out & 15)) return AF3_ERR_BAD_ARG;
  const int64_t blocks = (batch * n_q * (channels >> 3) + 255) / 256;
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  hipLaunchKernelGGL(gather_rows_add_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, src, rows, add, out, batch,
                     n_src, n_q, channels);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

int launch_ln_project3_gather(const bf16_t* x, const int* rows, const float* ln_w, const float* w, float* out,
                              int64_t batch, int64_t n_src, int64_t n_out, int channels, hipStream_t stream) {
  if (!x || !rows || !ln_w || !w || !out || batch <= 0 || n_src <= 0 || n_out <= 0) return AF3_ERR_BAD_ARG;
  if (channels != 128) return AF3_ERR_UNSUPPORTED;
  if ((uintptr_t)x & 15) return AF3_ERR_BAD_ARG;
  const int64_t blocks = (batch * n_out + 255) / 256;
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  hipLaunchKernelGGL(ln_project3_gather_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, rows, ln_w, w, out, batch,
                     n_src, n_out);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

int launch_atom_position_features(const float* pos, const int* rows, const float* w, const float* cond, void* out,
                                  int out_f32, int64_t batch, int64_t n_slots, int64_t n_q, int channels,
                                  hipStream_t stream) {
  if (!pos || !rows || !w || !cond || !out || batch <= 0 || n_slots <= 0 || n_q <= 0 || channels <= 0 || (channels & 7))
    return AF3_ERR_BAD_ARG;
  if (((uintptr_t)cond & 15) || ((uintptr_t)out & 15)) return AF3_ERR_BAD_ARG;
  const int64_t items = batch * n_q * (channels >> 3);
  const int64_t blocks = (items + 255) / 256;
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  const dim3 grid((unsigned)blocks), block(256);
  if (out_f32)
    hipLaunchKernelGGL(atom_position_features_kernel<float>, grid, block, 0, stream, pos, rows, w, cond,
                       static_cast<float*>(out), batch, n_slots, n_q, channels);
  else
    hipLaunchKernelGGL(atom_position_features_kernel<bf16_t>, grid, block, 0, stream, pos, rows, w, cond,
                       static_cast<bf16_t*>(out), batch, n_slots, n_q, channels);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

int launch_gathered_relu_mean(const bf16_t* src, const int* idx, const float* count, float* out, int64_t batch,
                              int64_t n_src, int64_t n_out, int slots, int channels, hipStream_t stream) {
  if (!src || !idx || !count || !out || batch <= 0 || n_src <= 0 || n_out <= 0 || slots <= 0 || slots > 32 ||
      channels <= 0 || (channels & 7))
    return AF3_ERR_BAD_ARG;
  if (((uintptr_t)src & 15) || ((uintptr_t)out & 15)) return AF3_ERR_BAD_ARG;
  const int64_t items = batch * n_out * (channels >> 3);
  const int64_t blocks = (items + 255) / 256;
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  const dim3 grid((unsigned)blocks), block(256);
  if (slots <= 8)
    hipLaunchKernelGGL(gathered_relu_mean_kernel<8>, grid, block, 0, stream, src, idx, count, out, batch, n_src, n_out, slots, channels);
  else if (slots <= 24)
    hipLaunchKernelGGL(gathered_relu_mean_kernel<24>, grid, block, 0, stream, src, idx, count, out, batch, n_src, n_out, slots, channels);
  else
    hipLaunchKernelGGL(gathered_relu_mean_kernel<32>, grid, block, 0, stream, src, idx, count, out, batch, n_src, n_out, slots, channels);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

int launch_transpose(const bf16_t* in, bf16_t* out, int64_t rows, int64_t cols, hipStream_t stream) {
  if (!in || !out || rows <= 0 || cols <= 0 || (rows & 7) || (cols & 7)) return AF3_ERR_BAD_ARG;
  if (((uintptr_t)in & 15) || ((uintptr_t)out & 15)) return AF3_ERR_BAD_ARG;
  const int64_t blocks = ((rows + TT - 1) / TT) * ((cols + TT - 1) / TT);
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  hipLaunchKernelGGL(transpose_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, in, out, rows, cols);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

int launch_softmax_rows(const float* x, const float* mask, bf16_t* y, int64_t rows, int cols, int64_t ldy,
                        hipStream_t stream) {
  if (!x || !y || rows <= 0 || cols <= 0 || ldy < cols) return AF3_ERR_BAD_ARG;
  const int64_t blocks = (rows + 3) / 4;
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  hipLaunchKernelGGL(softmax_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, mask, y, rows, cols, ldy);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

int launch_narrow_linear_f32(const float* x, const float* w, const float* res, float* y, int64_t rows, int k, int n_out,
                             int relu_in, hipStream_t stream) {
  if (!x || !w || !y || rows <= 0 || k <= 0 || k > 128 || (k & 3)) return AF3_ERR_BAD_ARG;
  if (n_out != 16 && n_out != 3) return AF3_ERR_UNSUPPORTED;
  if ((uintptr_t)x & 15) return AF3_ERR_BAD_ARG;
  const int64_t blocks = (rows + 255) / 256;
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  const dim3 grid((unsigned)blocks), block(256);
  if (n_out == 16) hipLaunchKernelGGL(narrow_linear_f32_kernel<16>, grid, block, 0, stream, x, w, res, y, rows, k, relu_in);
  else hipLaunchKernelGGL(narrow_linear_f32_kernel<3>, grid, block, 0, stream, x, w, res, y, rows, k, relu_in);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

int launch_atom_pair_logits(const float* x, const float* ln_w, const float* w, float* out, int64_t n_groups, int64_t group,
                            int n_blocks, int n_head, hipStream_t stream) {
  if (!x || !ln_w || !w || !out || n_groups <= 0 || group <= 0 || n_blocks <= 0 || n_head <= 0) return AF3_ERR_BAD_ARG;
  if (n_blocks * n_head > 32) return AF3_ERR_UNSUPPORTED;
  if ((uintptr_t)x & 15) return AF3_ERR_BAD_ARG;
  const int64_t rows = n_groups * group, blocks = (rows + 255) / 256;
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  hipLaunchKernelGGL(atom_pair_logits_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, ln_w, w, out, rows, group,
                     n_groups, n_blocks, n_head);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

int launch_atom_pair_cond(const float* row, const float* col, const float* tp, const int* tq, const int* tk, int n_tok,
                          const float* q_pos, const float* k_pos, const int* q_uid, const int* k_uid, const float* w_off,
                          const float* w_dist, const float* w_valid, const float* w1, const float* w2, const float* w3,
                          float* out, int64_t subsets, int queries, int keys, hipStream_t stream) {
  if (!row || !col || !q_pos || !k_pos || !q_uid || !k_uid || !w_off || !w_dist || !w_valid || !w1 || !w2 || !w3 || !out)
    return AF3_ERR_BAD_ARG;
  if (subsets <= 0 || queries <= 0 || keys <= 0) return AF3_ERR_BAD_ARG;
  if (tp && (!tq || !tk || n_tok <= 0)) return AF3_ERR_BAD_ARG;
  if (((uintptr_t)row & 15) || ((uintptr_t)col & 15) || ((uintptr_t)tp & 15) || ((uintptr_t)out & 15)) return AF3_ERR_BAD_ARG;
  AtomPairCondArgs a{row, col, tp, tq, tk, q_pos, k_pos, q_uid, k_uid, w_off, w_dist, w_valid, w1, w2, w3, out,
                     subsets, queries, keys, n_tok};
  const int64_t blocks = (subsets * queries * keys + 255) / 256;
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  hipLaunchKernelGGL(atom_pair_cond_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}
