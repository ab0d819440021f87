// Device helpers shared by the row-tile kernels of the 128-channel pair path:
// tile geometry, LayerNorm of a 128-pixel tile into LDS, weight staging, MFMA
// chunk products in "D form" (out[px][ch], lane owns a channel) or "T form"
// (out^T[ch][px], lane owns a pixel), and staged stores.
#pragma once
#include "common.h"

namespace {

constexpr int C = 128;    // pair channels
constexpr int TM = 128;   // positions per tile
constexpr int LDX = 136;  // LDS row stride (bf16) for [row][128] tiles: 272 B
constexpr int LDS_F = 132;  // LDS row stride (fp32) for staged output tiles

struct Tile {
  int o, r0, N;
  int64_t so, sr;  // pixel index = o * so + r * sr
  __device__ __forceinline__ int64_t pix(int p) const { return (int64_t)o * so + (int64_t)(r0 + p) * sr; }
  __device__ __forceinline__ bool valid(int p) const { return r0 + p < N; }
};

// `reverse`: walk the tiles from the last to the first.  A kernel that reads
// what the previous kernel has just written (and whose output the next kernel
// starts reading from the other end) finds the most recently written part
// still in the last-level cache when it starts there.
__device__ __forceinline__ Tile make_tile(int N, bool column_mode, bool reverse = false) {
  const int tiles_r = (N + TM - 1) / TM;
  Tile t;
  t.N = N;
  const unsigned bid = reverse ? gridDim.x - 1 - blockIdx.x : blockIdx.x;
  t.o = bid / tiles_r;
  t.r0 = (bid % tiles_r) * TM;
  t.so = column_mode ? 1 : N;
  t.sr = column_mode ? N : 1;
  return t;
}

// Eight consecutive fp32 parameters (LayerNorm weight / bias slice of a thread),
// or a constant when the pointer is null.
__device__ __forceinline__ void load_param8(const float* p, float fill, float* out) {
  if (p) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p);
    const f32x4 b = *reinterpret_cast<const f32x4*>(p + 4);
    out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
    out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = fill;
  }
}

// LayerNorm of one pixel's eight channels (the thread's share: 16 lanes cooperate on the
// pixel's statistics) -> packed bf16.
//
// This phase is vector arithmetic per element and a large share of every tile
// kernel's instructions, so the bf16 stream takes the short form: sum and sum of
// squares in one pass (variance = E[x^2] - mean^2 in fp32: the error relative to
// the variance is 1e-7 (1 + mean^2 / variance), and a bf16 tensor cannot hold a
// mean of more than ~2^8 standard deviations to begin with), normalisation as two
// FMAs per element (x * rstd - mean * rstd, then * w + b), and no per-element
// select when every pixel of the tile is in range.  The fp32 stream keeps the
// two-pass form.  Zero-padded channels (fewer than 128 real ones) add nothing to
// either sum; the two-pass form takes their pad * mean^2 out again.
template <typename TIO>
__device__ __forceinline__ u32x4 ln_pixel8(const typename Elem<TIO>::Raw& raw, const float* w, const float* b,
                                           bool skip_ln, float inv_c, float pad) {
  using E = Elem<TIO>;
  constexpr bool ONE_PASS = sizeof(TIO) == 2;
  float v[8], o[8];
  E::unpack_raw(raw, v);
  if (ONE_PASS) {
    float s = 0.f, q = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) { s += v[e]; q = fmaf(v[e], v[e], q); }
    const float mean = group16_sum(s) * inv_c;
    const float var = fmaxf(fmaf(group16_sum(q), inv_c, -mean * mean), 0.f);
    // (an already normalised input comes with w = 1, b = 0: scale 1 and shift 0 pass it through unchanged)
    const float rstd = skip_ln ? 1.f : rsqrtf(var + LN_EPS);
    const float shift = skip_ln ? 0.f : -mean * rstd;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = fmaf(fmaf(v[e], rstd, shift), w[e], b[e]);
  } else {
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) s += v[e];
    const float mean = group16_sum(s) * inv_c;
    float q = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) { const float d = v[e] - mean; q += d * d; }
    // (zero-padded channels, if any, each put mean^2 into the sum)
    const float rstd = rsqrtf((group16_sum(q) - pad * mean * mean) * inv_c + LN_EPS);
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = skip_ln ? v[e] : (v[e] - mean) * rstd * w[e] + b[e];
  }
  return pack8(o);
}

// LayerNorm of a tile of pixels from global memory into sX[p][c] (bf16).
// Thread (prow = tid / 16, chunk = tid % 16) handles channels 8*chunk..+7 of
// pixels prow, prow + 16, ...; 16 lanes cooperate on one pixel's statistics.
// Out-of-range pixels become zero rows.  The loads of a batch of pixels are
// unconditional (an out-of-range pixel re-reads the tile's first one) and all
// issued before any value is converted: a load under a lane mask, or one whose
// value is touched at once, costs a full memory round trip per pixel.
template <typename TIO>
__device__ __forceinline__ void load_ln_tile(const TIO* x, const Tile& t, const float* lnw,
                                             const float* lnb, bf16_t* sX, int tid, bool skip_ln = false,
                                             float inv_c = 1.f / C, float pad = 0.f) {
  using E = Elem<TIO>;
  constexpr int NB = E::kBatch;
  const int chunk = tid & 15, prow = tid >> 4;
  float w[8], b[8];
  load_param8(lnw ? lnw + chunk * 8 : nullptr, 1.f, w);
  load_param8(lnb ? lnb + chunk * 8 : nullptr, 0.f, b);
  const bool full = t.r0 + TM <= t.N;  // every pixel of the tile is in range (uniform over the workgroup)
#pragma unroll
  for (int base = 0; base < 8; base += NB) {
    typename E::Raw raw[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int p = (base + i) * 16 + prow;
      raw[i] = E::load_raw(x + t.pix(t.valid(p) ? p : 0) * C + chunk * 8);
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int p = (base + i) * 16 + prow;
      u32x4 pk = ln_pixel8<TIO>(raw[i], w, b, skip_ln, inv_c, pad);
      if (!full && !t.valid(p)) pk = u32x4{0u, 0u, 0u, 0u};
      *reinterpret_cast<u32x4*>(sX + p * LDX + chunk * 8) = pk;
    }
  }
}

// In-place LayerNorm of the rows of sX (bf16 in LDS), same thread mapping.
__device__ __forceinline__ void ln_inplace_tile(bf16_t* sX, const float* lnw, const float* lnb, int tid) {
  const int chunk = tid & 15, prow = tid >> 4;
  float w[8], b[8];
  load_param8(lnw + chunk * 8, 1.f, w);
  load_param8(lnb + chunk * 8, 0.f, b);
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int p = it * 16 + prow;
    float v[8];
    unpack8(*reinterpret_cast<const u32x4*>(sX + p * LDX + chunk * 8), v);
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) s += v[e];
    const float mean = group16_sum(s) * (1.f / C);
    float q = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) { const float d = v[e] - mean; q += d * d; }
    const float rstd = rsqrtf(group16_sum(q) * (1.f / C) + LN_EPS);
    float o[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (v[e] - mean) * rstd * w[e] + b[e];
    *reinterpret_cast<u32x4*>(sX + p * LDX + chunk * 8) = pack8(o);
  }
}

// Copy `rows` x 128 bf16 weights (row-major, contiguous) into sW[row][LDX].
__device__ __forceinline__ void load_w_rows(const bf16_t* gW, bf16_t* sW, int rows, int tid) {
  for (int idx = tid; idx < rows * 16; idx += 256) {
    const int row = idx >> 4, ch = idx & 15;
    *reinterpret_cast<u32x4*>(sW + row * LDX + ch * 8) =
        *reinterpret_cast<const u32x4*>(gW + row * C + ch * 8);
  }
}

// The wave's 32 pixels as 8 k-step fragments (k = 128 channels).
__device__ __forceinline__ void load_x_frags(const bf16_t* sX, int wave, int lane, bf16x8* xf) {
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) xf[ks] = lds_frag(sX, LDX, wave * 32, ks * 16, lane);
}

// acc[nt] = tile nt (32 weight rows) of  X * W^T  (D form) or  W * X^T  (T form)
template <bool TFORM, int NT>
__device__ __forceinline__ void mfma_chunk(const bf16x8* xf, const bf16_t* sW, int lane, f32x16* acc) {
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[nt][r] = 0.f;
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int ks = 0; ks < 8; ++ks)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const bf16x8 wf = lds_frag(sW, LDX, nt * 32, ks * 16, lane);
      acc[nt] = TFORM ? mfma32(wf, xf[ks], acc[nt]) : mfma32(xf[ks], wf, acc[nt]);
    }
  // Weight fragments are read four ahead of the MFMAs that use them (left to
  // itself the compiler reads each one right in front of its MFMA and waits).
  __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
  for (int i = 0; i < 8 * NT - 4; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
  }
  __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
  __builtin_amdgcn_sched_barrier(0);
}

// T-form accumulators (lane = pixel, 4 consecutive channels per register
// quad) -> fp32 staging tile sS[px][LDS_F].
__device__ __forceinline__ void stage_t_f32(const f32x16* acc, float* sS, int wave, int lane) {
  const int px = wave * 32 + (lane & 31);
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int ch = nt * 32 + 8 * g + 4 * (lane >> 5);
      f32x4 v = {acc[nt][4 * g], acc[nt][4 * g + 1], acc[nt][4 * g + 2], acc[nt][4 * g + 3]};
      *reinterpret_cast<f32x4*>(sS + px * LDS_F + ch) = v;
    }
}

// T-form accumulators -> bf16 staging tile sS[px][LDX]
__device__ __forceinline__ void stage_t_bf16(const f32x16* acc, bf16_t* sS, int wave, int lane) {
  const int px = wave * 32 + (lane & 31);
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int ch = nt * 32 + 8 * g + 4 * (lane >> 5);
      u32x2 v;
      v.x = pack2bf(acc[nt][4 * g], acc[nt][4 * g + 1]);
      v.y = pack2bf(acc[nt][4 * g + 2], acc[nt][4 * g + 3]);
      *reinterpret_cast<u32x2*>(sS + px * LDX + ch) = v;
    }
}

// Staged fp32 tile -> residual stream: out[pix] = (res ? res[pix] : 0) + tile.
// The residual rows of a batch of pixels are loaded (unconditionally, from a
// clamped pixel) before the batch's first store: out may alias res, so the
// compiler cannot move a load above a store on its own.
template <typename TIO>
__device__ __forceinline__ void store_tile_f32(const float* sS, const Tile& t, TIO* out, const TIO* res, int tid) {
  using E = Elem<TIO>;
  constexpr int NB = E::kBatch;
  const int chunk = tid & 15, prow = tid >> 4;
#pragma unroll
  for (int base = 0; base < 8; base += NB) {
    typename E::Raw raw[NB];
    if (res) {
#pragma unroll
      for (int i = 0; i < NB; ++i) {
        const int p = (base + i) * 16 + prow;
        raw[i] = E::load_raw(res + t.pix(t.valid(p) ? p : 0) * C + chunk * 8);
      }
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int p = (base + i) * 16 + prow;
      float v[8];
      const f32x4 a = *reinterpret_cast<const f32x4*>(sS + p * LDS_F + chunk * 8);
      const f32x4 b = *reinterpret_cast<const f32x4*>(sS + p * LDS_F + chunk * 8 + 4);
      v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
      if (res) {
        float rr[8];
        E::unpack_raw(raw[i], rr);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += rr[e];
      }
      if (t.valid(p)) E::store8(out + t.pix(p) * C + chunk * 8, v);
    }
  }
}


// 128 x 128 bf16 weight chunk held in registers between a global load and the
// LDS store, so the load overlaps the MFMA work on the previous chunk.
struct WChunkRegs {
  u32x4 r[8];
  // SWAP23: register row rho receives weight row swap23(rho) (bits 2 and 3 exchanged)
  template <bool SWAP23 = false>
  __device__ __forceinline__ void load(const bf16_t* gW, int tid) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int idx = tid + 256 * i, rho = idx >> 4;
      const int row = SWAP23 ? ((rho & ~12) | ((rho & 4) << 1) | ((rho & 8) >> 1)) : rho;
      r[i] = *reinterpret_cast<const u32x4*>(gW + row * C + (idx & 15) * 8);
    }
  }
  __device__ __forceinline__ void store(bf16_t* sW, int tid) const {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int idx = tid + 256 * i;
      *reinterpret_cast<u32x4*>(sW + (idx >> 4) * LDX + (idx & 15) * 8) = r[i];
    }
  }
};

}  // namespace
