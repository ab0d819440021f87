// Triangle attention, the fast path: the projection kernel.  It produces, in one
// pass over the pair tensor, everything the attention core (triattn_core.hip)
// reads, in the layouts it wants (described in kernels.h): head-major q (scaled)
// and k, V transposed with the key order the core's MFMA fragments use, and the
// fp16 pair bias in the order of the core's MFMA fragments.  (The output gate is
// computed where it is used, by attn_out_kernel.)
#include "common.h"
#include "kernels.h"
#include <type_traits>

#include "tile_common.h"

namespace {

constexpr int H = 4, D = 32;

// ============================================================================
// projections: LN -> q (scaled), k (position-major) and v (channel-major),
// + pair-bias heads
// ============================================================================
template <typename TIO>
__global__ __launch_bounds__(256, 3) void triattn_proj_kernel(TriAttnProjArgs a) {
  // 34.8 KB + 17.4 KB of LDS and at most 168 registers: three workgroups per CU.  The kernel is a chain of
  // short dependent phases (load, LayerNorm, MFMA, stage, store), so what it needs is company.
  __shared__ __attribute__((aligned(16))) bf16_t sX[TM * LDX];  // LN tile, then staging
  __shared__ __attribute__((aligned(16))) bf16_t sW[64 * LDX];  // 64 weight rows at a time
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // (b, s) = (o, r): for the transposed operator a tile is a column segment
  // last tile first: the pair tensor was written front to back by the operator
  // before this one, and the attention core that follows starts with row 0,
  // which is then the freshest part of q / k / v (measured: 1.4 % of the block)
  const Tile t = make_tile(a.N, a.transpose != 0, true);
  const TIO* x = reinterpret_cast<const TIO*>(a.pair);
  // Step s = 2 * chunk + half: weight rows 64 half .. + 63 of chunk s / 2 (chunks q, k, v of w_qkvg),
  // four 16-byte pieces per thread; the 32 (padded) pair-bias rows ride in the same registers.
  u32x4 wr[4];
  auto wload = [&](int s) {
    const bf16_t* base = a.w_qkvg + (int64_t)s * 64 * C;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + 256 * i;
      wr[i] = *reinterpret_cast<const u32x4*>(base + (idx >> 4) * C + (idx & 15) * 8);
    }
  };
  auto wload_bias = [&]() {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int idx = tid + 256 * i;
      wr[i] = *reinterpret_cast<const u32x4*>(a.w_bias + (idx >> 4) * C + (idx & 15) * 8);
    }
  };
  auto wstore = [&](int n) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + 256 * i;
      if (i < n) *reinterpret_cast<u32x4*>(sW + (idx >> 4) * LDX + (idx & 15) * 8) = wr[i];
    }
  };
  wload(0);
  load_ln_tile<TIO>(x, t, a.ln_w, a.ln_b, sX, tid, a.skip_ln != 0, a.lw.inv_c, a.lw.pad);
  wstore(4);
  lds_barrier();
  bf16x8 xf[8];
  load_x_frags(sX, wave, lane, xf);
  lds_barrier();  // sX is free from here on: it becomes the staging tile

  const int64_t bh0 = (int64_t)t.o * H;  // (b * H + h) for h = 0
  // v takes the channel-major route.  The step index is a compile-time constant of the body: with a
  // run-time index the compiler evaluates the sigmoid for every chunk and selects.
  auto do_step = [&](auto step_c) {
    constexpr int step = decltype(step_c)::value, chunk = step >> 1, pairt = step & 1;
    // The next weights are requested BEFORE this chunk's results are stored:
    // vector memory operations retire in order, so a load issued behind the
    // stores would make its consumer wait for the stores' round trip to HBM.
    if (step < 5) wload(step + 1);
    else if (a.n_bias > 0) wload_bias();
    {
      f32x16 acc[2];
      if (chunk == 2) {
        // v: D form, lane owns channel (lane & 31) of a tile, registers walk pixels
        mfma_chunk<false, 2>(xf, sW, lane, acc);
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
          const int ch = (pairt * 2 + nt) * 32 + (lane & 31);
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int p0 = wave * 32 + 8 * g + 4 * (lane >> 5);
            u32x2 pk;
            pk.x = pack2bf(acc[nt][4 * g], acc[nt][4 * g + 1]);
            pk.y = pack2bf(acc[nt][4 * g + 2], acc[nt][4 * g + 3]);
            *reinterpret_cast<u32x2*>(sX + ch * LDX + tri_vt_pos(p0)) = pk;
          }
        }
      } else {
        mfma_chunk<true, 2>(xf, sW, lane, acc);
        const int px = wave * 32 + (lane & 31);
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float y = acc[nt][4 * g + e];
              v[e] = chunk == 0 ? y * a.q_scale : y;
            }
            const int ch = (pairt * 2 + nt) * 32 + 8 * g + 4 * (lane >> 5);
            u32x2 pk;
            pk.x = pack2bf(v[0], v[1]);
            pk.y = pack2bf(v[2], v[3]);
            *reinterpret_cast<u32x2*>(sX + px * LDX + ch) = pk;
          }
      }
    }
    lds_barrier();  // staging visible; every wave is done with sW
    if (step < 5) wstore(4);
    else if (a.n_bias > 0) wstore(2);
    if (pairt == 1) {
      // both halves of the chunk are staged: 128 channels per position go out
      if (chunk == 2) {
        // Vt[(b*H + h)*32 + d][tri_vt_pos(s)]: per channel 128 consecutive columns (the quads of
        // a 16-key group were swapped on their way into the staging tile)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int idx = tid + 256 * i, ch = idx >> 4, pc = idx & 15;
          const int r = t.r0 + pc * 8;
          if (r < a.ldn)
            *reinterpret_cast<u32x4*>(a.vt + (bh0 * D + ch) * a.ldn + r) =
                *reinterpret_cast<const u32x4*>(sX + ch * LDX + pc * 8);
        }
      } else {
        bf16_t* plane = chunk == 0 ? a.q : a.k;
        const int ck = tid & 15, prow = tid >> 4;
        const int h = ck >> 2, part = ck & 3;
#pragma unroll
        for (int it = 0; it < 8; ++it) {
          const int p = it * 16 + prow;
          if (t.valid(p))
            *reinterpret_cast<u32x4*>(plane + ((bh0 + h) * a.N + t.r0 + p) * D + part * 8) =
                *reinterpret_cast<const u32x4*>(sX + p * LDX + ck * 8);
        }
      }
    }
    lds_barrier();
  };
  do_step(std::integral_constant<int, 0>{});
  do_step(std::integral_constant<int, 1>{});
  do_step(std::integral_constant<int, 2>{});
  do_step(std::integral_constant<int, 3>{});
  do_step(std::integral_constant<int, 4>{});
  do_step(std::integral_constant<int, 5>{});

  // pair-bias heads (T form: lane = pixel, rows = heads): bias[h][q][k] with
  // (q, k) the pixel's own (row, col) in the un-transposed pair tensor
  if (a.n_bias > 0) {
    f32x16 acc[1];
    mfma_chunk<true, 1>(xf, sW, lane, acc);
    if ((lane >> 5) == 0) {  // heads 0..3 are accumulator rows 0..3: registers 0..3 of the low half
      const int p = wave * 32 + lane;
      const int r = t.r0 + p;
      const int kpad = (int)tri_bias_ktiles(a.N) * 64;  // keys N..kpad-1 are padding: zero bias
      if (!a.transpose) {
        // q = o, k = r
        if (r < kpad) {
#pragma unroll
          for (int h = 0; h < H; ++h)
            a.bias[tri_bias_offset(a.N, h, t.o, r)] = f2h_sat(t.valid(p) ? acc[0][h] * a.bias_scale : 0.f);
        }
      } else if (t.valid(p)) {
        // q = r, k = o
#pragma unroll
        for (int h = 0; h < H; ++h) {
          a.bias[tri_bias_offset(a.N, h, r, t.o)] = f2h_sat(acc[0][h] * a.bias_scale);
          if (t.o == a.N - 1)
            for (int k = a.N; k < kpad; ++k) a.bias[tri_bias_offset(a.N, h, r, k)] = 0;
        }
      }
    }
  }
}

bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

int launch_triattn_proj(const TriAttnProjArgs& a, hipStream_t stream) {
  if (a.N <= 0 || !a.pair || !a.w_qkvg || !a.q || !a.k || !a.vt) return AF3_ERR_BAD_ARG;
  if (a.ldn < a.N || (a.ldn & 15)) return AF3_ERR_BAD_ARG;
  if (a.n_bias != 0 && (a.n_bias != H || !a.w_bias || !a.bias)) return AF3_ERR_BAD_ARG;
  if (!al16(a.pair) || !al16(a.w_qkvg) || !al16(a.w_bias) || !al16(a.q) || !al16(a.k) || !al16(a.vt) ||
      !al16(a.bias))
    return AF3_ERR_BAD_ARG;
  const int64_t tiles = (int64_t)a.N * ((a.N + TM - 1) / TM);
  if (tiles > 0x7fffffff) return AF3_ERR_BAD_ARG;
  if (a.io_f32) hipLaunchKernelGGL(triattn_proj_kernel<float>, dim3((unsigned)tiles), dim3(256), 0, stream, a);
  else hipLaunchKernelGGL(triattn_proj_kernel<bf16_t>, dim3((unsigned)tiles), dim3(256), 0, stream, a);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}
