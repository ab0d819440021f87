// Shared device helpers for the gfx950 (CDNA4) kernels: bf16 conversion, MFMA
// fragment conventions, wave reductions and LDS tile geometry.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define AF3_OK 0
#define AF3_ERR_BAD_ARG (-1)
#define AF3_ERR_WORKSPACE (-2)
#define AF3_ERR_LAUNCH (-3)
#define AF3_ERR_UNSUPPORTED (-4)
#define AF3_ERR_TOO_LARGE (-5)

typedef uint16_t bf16_t;  // raw bf16 bits in memory

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define WAVE 64

// ----------------------------------------------------------------------------
// bf16 <-> fp32 (round to nearest even; NaN kept quiet)
// ----------------------------------------------------------------------------
__device__ __forceinline__ float bf2f(bf16_t h) {
  return __uint_as_float(((uint32_t)h) << 16);
}
__device__ __forceinline__ bf16_t f2bf(float f) {
  return __builtin_bit_cast(bf16_t, (__bf16)f);
}
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
// two floats -> packed bf16 pair, round to nearest even (one v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack2bf(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ float bflo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bfhi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// fp32 -> fp16 bits, round to nearest even, saturating at the largest finite fp16
__device__ __forceinline__ uint16_t f2h_sat(float f) {
  f = fminf(fmaxf(f, -65504.f), 65504.f);
  return __builtin_bit_cast(uint16_t, (_Float16)f);
}
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
// 8 consecutive bf16 (16 bytes) <-> 8 floats
__device__ __forceinline__ void unpack8(const u32x4 v, float* f) {
  f[0] = bflo(v.x); f[1] = bfhi(v.x); f[2] = bflo(v.y); f[3] = bfhi(v.y);
  f[4] = bflo(v.z); f[5] = bfhi(v.z); f[6] = bflo(v.w); f[7] = bfhi(v.w);
}
__device__ __forceinline__ u32x4 pack8(const float* f) {
  u32x4 v;
  v.x = pack2bf(f[0], f[1]); v.y = pack2bf(f[2], f[3]);
  v.z = pack2bf(f[4], f[5]); v.w = pack2bf(f[6], f[7]);
  return v;
}

// Load / store 8 consecutive channels of the residual stream, which may be
// held as bf16 or fp32.
template <typename T> struct Elem;
template <> struct Elem<bf16_t> {
  static __device__ __forceinline__ void load8(const bf16_t* p, float* f) {
    unpack8(*reinterpret_cast<const u32x4*>(p), f);
  }
  static __device__ __forceinline__ void store8(bf16_t* p, const float* f) {
    *reinterpret_cast<u32x4*>(p) = pack8(f);
  }
  static __device__ __forceinline__ float load(const bf16_t* p) { return bf2f(*p); }
  static __device__ __forceinline__ void store(bf16_t* p, float v) { *p = f2bf(v); }
  // 8 elements as loaded, conversion deferred: lets a kernel put a batch of
  // loads in flight before the first value is touched
  struct Raw { u32x4 v; };
  static constexpr int kBatch = 8;  // 8-element groups to keep in flight at a time (4 VGPRs each)
  static __device__ __forceinline__ Raw load_raw(const bf16_t* p) { return Raw{*reinterpret_cast<const u32x4*>(p)}; }
  static __device__ __forceinline__ void unpack_raw(const Raw& r, float* f) { unpack8(r.v, f); }
};
template <> struct Elem<float> {
  static __device__ __forceinline__ void load8(const float* p, float* f) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p);
    const f32x4 b = *reinterpret_cast<const f32x4*>(p + 4);
    f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w;
    f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
  }
  static __device__ __forceinline__ void store8(float* p, const float* f) {
    f32x4 a = {f[0], f[1], f[2], f[3]}, b = {f[4], f[5], f[6], f[7]};
    *reinterpret_cast<f32x4*>(p) = a;
    *reinterpret_cast<f32x4*>(p + 4) = b;
  }
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
  struct Raw { f32x4 a, b; };
  static constexpr int kBatch = 4;  // 8 VGPRs per group
  static __device__ __forceinline__ Raw load_raw(const float* p) {
    return Raw{*reinterpret_cast<const f32x4*>(p), *reinterpret_cast<const f32x4*>(p + 4)};
  }
  static __device__ __forceinline__ void unpack_raw(const Raw& r, float* f) {
    f[0] = r.a.x; f[1] = r.a.y; f[2] = r.a.z; f[3] = r.a.w;
    f[4] = r.b.x; f[5] = r.b.y; f[6] = r.b.z; f[7] = r.b.w;
  }
};

// sigmoid through the hardware exp2 / reciprocal (about 1 ulp each): four
// instructions instead of the ~15 of an IEEE division.  exp2 overflows to +inf
// for very negative x and rcp(inf) = 0, as it should.
__device__ __forceinline__ float sigmoidf_(float x) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}

// ----------------------------------------------------------------------------
// MFMA 32x32x16 bf16 (D = A[32xK16] * B[K16x32] + C), wave64.
//   A fragment: lane l holds A[row = l & 31][k = 8*(l >> 5) .. +7]
//   B fragment: lane l holds B[k = 8*(l >> 5) .. +7][col = l & 31]
//   C/D       : lane l, register r holds D[row = 8*(r >> 2) + 4*(l >> 5) + (r & 3)][col = l & 31]
// Both fragments are "8 consecutive k of one row/col", so an operand stored
// k-contiguous ([row][k]) is read with one 16-byte load per fragment.
// ----------------------------------------------------------------------------
__device__ __forceinline__ f32x16 mfma32(const bf16x8 a, const bf16x8 b, const f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mfma32_f16(const f16x8 a, const f16x8 b, const f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f16x8 as_frag_f16(const u32x4 v) { return __builtin_bit_cast(f16x8, v); }
__device__ __forceinline__ bf16x8 as_frag(const u32x4 v) {
  return __builtin_bit_cast(bf16x8, v);
}
__device__ __forceinline__ int acc_row(int r, int lane) {
  return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
}

// 16-byte fragment read from an LDS tile stored [row][ld] (bf16, k-contiguous)
__device__ __forceinline__ bf16x8 lds_frag(const bf16_t* tile, int ld, int row0, int k0, int lane) {
  const bf16_t* p = tile + (row0 + (lane & 31)) * ld + k0 + 8 * (lane >> 5);
  return as_frag(*reinterpret_cast<const u32x4*>(p));
}

// ----------------------------------------------------------------------------
// reductions over groups of 16 / 64 lanes
// ----------------------------------------------------------------------------
// DPP lane permutations inside a row of 16 lanes (no LDS crossbar traffic)
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// sum over each aligned group of 16 lanes, result in every lane of the group:
// quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_ror:4, row_ror:8
__device__ __forceinline__ float group16_sum(float v) {
  v += dpp_mov<0xB1>(v); v += dpp_mov<0x4E>(v);
  v += dpp_mov<0x124>(v); v += dpp_mov<0x128>(v);
  return v;
}
// Exchange with the other half of the wave (lane l <-> lane l ^ 32) through
// ds_bpermute with the byte address computed once per kernel:
//   const int xaddr = half_swap_addr();  ...  other = half_swap(xaddr, mine);
__device__ __forceinline__ int half_swap_addr() { return ((int)(threadIdx.x & 63) ^ 32) << 2; }
__device__ __forceinline__ float half_swap(int xaddr, float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(xaddr, __builtin_bit_cast(int, v)));
}
__device__ __forceinline__ float wave_sum(float v) {
  v = group16_sum(v);
  v += __shfl_xor(v, 16); v += __shfl_xor(v, 32);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
  for (int m = 1; m < 64; m <<= 1) v = fmaxf(v, __shfl_xor(v, m));
  return v;
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits
// for every outstanding global load and STORE of the wave (vmcnt(0)), which
// exposes the full HBM write latency at each barrier of a kernel that streams
// results out while it keeps computing.  None of the kernels here passes data
// between threads through global memory, so waiting for LDS alone is enough.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

#define LN_EPS 1e-5f
