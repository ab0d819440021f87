// Row-tile kernels of the 128-channel pair path.
//
// Every kernel here walks the [N, N, 128] pair tensor in tiles of 128
// consecutive positions along one axis (a row segment, or a column segment for
// the transposed operators), keeps the tile's LayerNorm-ed activations in LDS /
// registers as bf16 MFMA fragments and multiplies them with 128x128 weight
// chunks streamed through LDS.  They are HBM-bound (one read of the pair tensor,
// one write of each product) except the SwiGLU transition, which is MFMA-bound.
//
//   trimul_prologue  LN -> [proj|gate] -> mask * sigmoid -> a, b channel-major
//   trimul_epilogue  channel-major contraction result -> LN -> out-proj ->
//                    * sigmoid(LN(x) Wgl^T) -> (+ residual)
//   attn_proj        LN -> q (scaled), k, v, sigmoid gate, + pair-bias heads
//   attn_out         attention output * sigmoid(LN(x) Wg^T) -> out-proj -> (+ residual)
//   transition       LN -> W1 -> silu(a) * b -> W2 -> (+ residual), hidden in registers
//
// MFMA orientation: "D form" computes out[px][ch] with the pixel fragments as
// the A operand (a lane then owns one channel and 16 pixels), "T form" computes
// out^T[ch][px] with the weight rows as A (a lane owns one pixel and groups of
// 4 consecutive channels).  D form feeds channel-major stores, T form feeds
// pixel-major stores; the fragments are the same registers in both.
#include <type_traits>

#include "common.h"
#include "kernels.h"
#include "tile_common.h"

namespace {

// ============================================================================
// triangle multiplication, prologue
// ============================================================================
template <typename TIO>
__global__ __launch_bounds__(256, 3) void trimul_prologue_kernel(TriMulArgs a) {
  // 34.8 KB + 17.4 KB + 0.5 KB of LDS and at most 168 registers: three workgroups per CU.
  //
  // Eight steps of 64 weight rows (32 projection rows and the 32 matching gate rows) per tile.  A wave
  // runs them as a software pipeline: the 16 MFMAs of step s are issued one by one with, behind each, the
  // gating arithmetic (mask * proj * sigmoid(gate), packing, staging) of one register pair of step s - 1.
  // Inside one wave the matrix unit works while the wave goes on issuing vector instructions; between
  // waves of a SIMD it does not, so phases run back to back cost the sum of the two.  One barrier per step:
  // the weights and the staged results are double-buffered.
  __shared__ __attribute__((aligned(16))) bf16_t sX[TM * LDX];  // LN tile; then [S0 | S1 | W odd steps]
  __shared__ __attribute__((aligned(16))) bf16_t sW0[64 * LDX];  // weights of the even steps
  __shared__ float sMask[TM];
  static_assert(2 * 32 * LDX + 64 * LDX <= TM * LDX, "staging buffers and the second weight buffer fit the LN tile");
  bf16_t* const sS0 = sX;
  bf16_t* const sS1 = sX + 32 * LDX;
  bf16_t* const sW1 = sX + 64 * LDX;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // outgoing: tiles run along k for fixed i (a[c][i][k]); incoming: along k for
  // fixed j, i.e. a column segment of the pair tensor (a'[c][j][k] = a[k][j][c]).
  const Tile t = make_tile(a.N, !a.outgoing);
  const TIO* x = reinterpret_cast<const TIO*>(a.pair);

  // Weight chunks in memory: [P(64 ch) | G(64 ch)] for a ch 0-63, a ch 64-127, b ch 0-63, b ch 64-127.
  // Step s = 2 * chunk + half takes projection rows 32 half .. +31 and gate rows 64 + 32 half .. +31 of
  // its chunk: 64 rows x 128, four 16-byte pieces per thread.
  u32x4 wr[4];
  auto wload = [&](int s) {
    const bf16_t* base = a.w_pg + ((int64_t)(s >> 1) * TM + (s & 1) * 32) * C;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + 256 * i, row = idx >> 4;  // 0..63
      wr[i] = *reinterpret_cast<const u32x4*>(base + ((row & 31) + (row >> 5) * 64) * C + (idx & 15) * 8);
    }
  };
  auto wstore = [&](bf16_t* dst) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + 256 * i;
      *reinterpret_cast<u32x4*>(dst + (idx >> 4) * LDX + (idx & 15) * 8) = wr[i];
    }
  };
  const float mk = tid < TM && t.valid(tid) ? (a.mask ? a.mask[t.pix(tid)] : 1.f) : 0.f;
  if (!__syncthreads_or(mk != 0.f)) {
    // Every position of the tile is masked (padding): a' and b' are zero there
    // whatever the activations are.  Write the zeros and skip the rest.
    const u32x4 z = {0, 0, 0, 0};
    for (int idx = tid; idx < 2 * C * 16; idx += 256) {
      const int op = idx >> 11, ch = (idx >> 4) & (C - 1), r = t.r0 + (idx & 15) * 8;
      if (r < a.Np)
        *reinterpret_cast<u32x4*>((op ? a.b_buf : a.a_buf) + ((int64_t)ch * a.N + t.o) * a.Np + r) = z;
    }
    return;
  }
  wload(0);
  if (tid < TM) sMask[tid] = mk;
  load_ln_tile<TIO>(x, t, a.ln_in_w, a.ln_in_b, sX, tid, false, a.lw.inv_c, a.lw.pad);
  wstore(sW0);
  wload(1);
  lds_barrier();
  bf16x8 xf[8];
  load_x_frags(sX, wave, lane, xf);
  lds_barrier();  // sX is free from here on
  wstore(sW1);    // W_1
  wload(2);

  f32x16 zero16;
#pragma unroll
  for (int r = 0; r < 16; ++r) zero16[r] = 0.f;
  f32x16 accA[2], accB[2];  // [0] projection, [1] gate; A: even steps, B: odd steps
  const int ch = lane & 31;

  // Step S (0..8): the MFMAs of step S (S < 8) into `cur`, the gating of step S - 1 (S > 0) out of `prev`.
  auto step = [&](auto step_c, f32x16* cur, f32x16* prev) {
    constexpr int S = decltype(step_c)::value;
    const bf16_t* w = (S & 1) ? sW1 : sW0;                    // W_S
    bf16_t* stage = ((S - 1) & 1) ? sS1 : sS0;                // staging of step S - 1
    // results of step S - 2, complete since the last barrier: 32 channels x 128 positions, two 16-byte
    // pieces per thread, requested from LDS now and sent out further down
    u32x4 outv[2];
    if (S >= 2) {
      const bf16_t* done = ((S - 2) & 1) ? sS1 : sS0;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int idx = tid + 256 * i;
        outv[i] = *reinterpret_cast<const u32x4*>(done + (idx >> 4) * LDX + (idx & 15) * 8);
      }
    }
    bf16x8 wf[3];  // weight fragments, read two MFMAs ahead
    auto frag = [&](int m) { return lds_frag(w, LDX, (m & 1) * 32, (m >> 1) * 16, lane); };  // MFMA m: k-step m / 2, tile m % 2
    if (S < 8) {
      wf[0] = frag(0);
      wf[1] = frag(1);
    }
    f32x4 m4 = {0.f, 0.f, 0.f, 0.f};
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < 16; ++m) {
      if (S > 0 && (m & 3) == 0)  // the masks of pixels p0 .. p0 + 3, p0 = wave * 32 + 8 (m >> 2) + 4 hh
        m4 = *reinterpret_cast<const f32x4*>(sMask + wave * 32 + 2 * m + 4 * (lane >> 5));
      if (S < 8) {
        if (m + 2 < 16) wf[(m + 2) % 3] = frag(m + 2);
        cur[m & 1] = mfma32(xf[m >> 1], wf[m % 3], m < 2 ? zero16 : cur[m & 1]);
      }
      if (S > 0) {
        // register m of the previous step: pixel p0 + (m & 3), p0 = wave * 32 + 8 (m >> 2) + 4 hh
        float v = prev[0][m] * m4[m & 3] * sigmoidf_(prev[1][m]);
        asm volatile("" : "+v"(v));  // keeps the arithmetic in this group
        prev[0][m] = v;
        if ((m & 3) == 3) {
          const int g = m >> 2;
          const int p0 = wave * 32 + 8 * g + 4 * (lane >> 5);
          u32x2 pk;
          pk.x = pack2bf(prev[0][4 * g], prev[0][4 * g + 1]);
          pk.y = pack2bf(prev[0][4 * g + 2], prev[0][4 * g + 3]);
          *reinterpret_cast<u32x2*>(stage + ch * LDX + p0) = pk;
        }
      }
      if (m == 7) {
        // half way: the next weights go to LDS (the buffer of step S + 1 was last read in step S - 1), the
        // ones after them are requested, and step S - 2's results leave
        if (S >= 1 && S + 1 < 8) {
          wstore((S + 1) & 1 ? sW1 : sW0);
          if (S + 2 < 8) wload(S + 2);
        }
        if (S >= 2) {
          constexpr int SO = S >= 2 ? S - 2 : 0;
          bf16_t* dst = (SO < 4 ? a.a_buf : a.b_buf) + ((int64_t)(((SO >> 1) & 1) * 64 + (SO & 1) * 32) * a.N + t.o) * a.Np;
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const int idx = tid + 256 * i, c2 = idx >> 4, pc = idx & 15;
            const int r = t.r0 + pc * 8;
            if (r < a.Np) *reinterpret_cast<u32x4*>(dst + (int64_t)c2 * a.N * a.Np + r) = outv[i];
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    lds_barrier();
  };
  step(std::integral_constant<int, 0>{}, accA, accB);
  step(std::integral_constant<int, 1>{}, accB, accA);
  step(std::integral_constant<int, 2>{}, accA, accB);
  step(std::integral_constant<int, 3>{}, accB, accA);
  step(std::integral_constant<int, 4>{}, accA, accB);
  step(std::integral_constant<int, 5>{}, accB, accA);
  step(std::integral_constant<int, 6>{}, accA, accB);
  step(std::integral_constant<int, 7>{}, accB, accA);
  step(std::integral_constant<int, 8>{}, accA, accB);  // gating of step 7, results of step 6
  {
    // results of step 7
    bf16_t* dst = a.b_buf + ((int64_t)(64 + 32) * a.N + t.o) * a.Np;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int idx = tid + 256 * i, c2 = idx >> 4, pc = idx & 15;
      const int r = t.r0 + pc * 8;
      if (r < a.Np)
        *reinterpret_cast<u32x4*>(dst + (int64_t)c2 * a.N * a.Np + r) =
            *reinterpret_cast<const u32x4*>(sS1 + c2 * LDX + pc * 8);
    }
  }
}

// ============================================================================
// triangle multiplication, epilogue
// ============================================================================
template <typename TIO>
__global__ __launch_bounds__(256, 2) void trimul_epilogue_kernel(TriMulArgs a) {
  __shared__ __attribute__((aligned(16))) bf16_t smem[2 * TM * LDX];
  bf16_t* sX = smem;
  bf16_t* sW = smem + TM * LDX;
  float* sS = reinterpret_cast<float*>(smem);  // [TM][LDS_F] fp32 over both, after the last MFMA
  static_assert(TM * LDS_F * 4 <= 2 * TM * LDX * 2, "staging tile must fit");
  __shared__ __attribute__((aligned(16))) float sP[2 * C];  // center LayerNorm weight | bias
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const Tile t = make_tile(a.N, false);
  const TIO* x = reinterpret_cast<const TIO*>(a.pair);

  // everything this tile needs from memory is requested up front
  WChunkRegs wr;
  wr.load(a.w_gl, tid);
  u32x4 rt[8];  // contraction result t[c][i][j0 + 8 pc ..], c = 16 it + tid / 16
  const int pc = tid & 15, crow = tid >> 4;
  // (a chunk that starts past the row's end re-reads the tile's first one; its pixels are zeroed later)
  const int j_chunk = t.r0 + pc * 8 < a.Np ? t.r0 + pc * 8 : t.r0;
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    // (channels past the valid ones were not contracted: their rows hold whatever the workspace held;
    // the load goes to a valid channel's row instead and is replaced by zeros below)
    const int c = it * 16 + crow;
    rt[it] = *reinterpret_cast<const u32x4*>(a.t_buf + ((int64_t)(c < a.valid_c ? c : 0) * a.N + t.o) * a.Np + j_chunk);
  }

  // 1. output gate from the LayerNorm-ed input: sigmoid(LN(x) Wgl^T), T form, kept in registers
  load_ln_tile<TIO>(x, t, a.ln_in_w, a.ln_in_b, sX, tid, false, a.lw.inv_c, a.lw.pad);
  wr.store(sW, tid);
  wr.load(a.w_out, tid);
  lds_barrier();
  bf16x8 xf[8];
  load_x_frags(sX, wave, lane, xf);
  f32x16 gate[4];
  mfma_chunk<true, 4>(xf, sW, lane, gate);
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int r = 0; r < 16; ++r) gate[nt][r] = sigmoidf_(gate[nt][r]);
  lds_barrier();

  // 2. center LayerNorm of the contraction result, without a transposed copy:
  // the channel-major chunks go to LDS as they are (sT[c][j], 16-byte stores),
  // and every lane gathers, for its own pixel, exactly the 64 channels that
  // its eight MFMA B-fragments hold (channels 16 ks + 8 hh + e; the other half
  // of the wave holds the other 64 of the same pixel).  Lanes of a half-wave
  // read consecutive pixels of one channel row: conflict-free, where a
  // transposing 2-byte scatter would put a whole wave on two banks.
  bf16_t* sT = sX;
#pragma unroll
  for (int it = 0; it < 8; ++it)
    *reinterpret_cast<u32x4*>(sT + (it * 16 + crow) * LDX + pc * 8) = it * 16 + crow < a.valid_c ? rt[it] : u32x4{0u, 0u, 0u, 0u};
  wr.store(sW, tid);
  if (tid < C) {
    sP[tid] = a.ln_c_w[tid];
    sP[C + tid] = a.ln_c_b[tid];
  }
  lds_barrier();
  {
    const int j = lane & 31, hh = lane >> 5;
    const int px = wave * 32 + j;
    const int xaddr = half_swap_addr();
    float v[8][8];
    float s1 = 0.f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        v[ks][e] = bf2f(sT[(16 * ks + 8 * hh + e) * LDX + px]);
        s1 += v[ks][e];
      }
    s1 += half_swap(xaddr, s1);
    const float mean = s1 * a.lw.inv_c;
    float s2 = 0.f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
#pragma unroll
      for (int e = 0; e < 8; ++e) { const float d = v[ks][e] - mean; s2 += d * d; }
    s2 += half_swap(xaddr, s2);
    const float rstd = rsqrtf((s2 - a.lw.pad * mean * mean) * a.lw.inv_c + LN_EPS);
    const bool ok = t.valid(px);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const f32x4 w0 = *reinterpret_cast<const f32x4*>(sP + 16 * ks + 8 * hh);
      const f32x4 w1 = *reinterpret_cast<const f32x4*>(sP + 16 * ks + 8 * hh + 4);
      const f32x4 b0 = *reinterpret_cast<const f32x4*>(sP + C + 16 * ks + 8 * hh);
      const f32x4 b1 = *reinterpret_cast<const f32x4*>(sP + C + 16 * ks + 8 * hh + 4);
      const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
      const float bb[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = ok ? (v[ks][e] - mean) * rstd * w[e] + bb[e] : 0.f;
      xf[ks] = as_frag(pack8(o));
    }
  }
  f32x16 acc[4];
  mfma_chunk<true, 4>(xf, sW, lane, acc);
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[nt][r] *= gate[nt][r];
  lds_barrier();
  stage_t_f32(acc, sS, wave, lane);
  lds_barrier();
  store_tile_f32<TIO>(sS, t, reinterpret_cast<TIO*>(a.out), a.residual ? x : nullptr, tid);
}

// ============================================================================
// triangle attention: projections
// ============================================================================
template <typename TIO>
__global__ __launch_bounds__(256, 2) void attn_proj_kernel(AttnProjArgs a) {
  __shared__ __attribute__((aligned(16))) bf16_t sX[TM * LDX];
  __shared__ __attribute__((aligned(16))) bf16_t sW[TM * LDX];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // (b, s) = (o, r): for the transposed operator a tile is a column segment
  const Tile t = make_tile(a.N, a.transpose != 0);
  const TIO* x = reinterpret_cast<const TIO*>(a.pair);
  load_ln_tile<TIO>(x, t, a.ln_w, a.ln_b, sX, tid, a.skip_ln != 0, a.lw.inv_c, a.lw.pad);
  lds_barrier();
  bf16x8 xf[8];
  load_x_frags(sX, wave, lane, xf);

  for (int chunk = 0; chunk < a.n_chunks; ++chunk) {
    load_w_rows(a.w_main + (int64_t)chunk * TM * C, sW, TM, tid);
    lds_barrier();
    f32x16 acc[4];
    mfma_chunk<true, 4>(xf, sW, lane, acc);
    const int op = (a.chunk_ops >> (4 * chunk)) & 15;
    if (op == SEG_BIAS_SCALE) {
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[nt][r] *= a.q_scale;
    } else if (op == SEG_SIGMOID) {
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[nt][r] = sigmoidf_(acc[nt][r]);
    }
    lds_barrier();
    stage_t_bf16(acc, sW, wave, lane);
    lds_barrier();
    const int ck = tid & 15, prow = tid >> 4;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int p = it * 16 + prow;
      if (t.valid(p))
        *reinterpret_cast<u32x4*>(a.out_main + ((int64_t)t.o * a.N + t.r0 + p) * a.ld_main + chunk * C + ck * 8) =
            *reinterpret_cast<const u32x4*>(sW + p * LDX + ck * 8);
    }
    lds_barrier();
  }

  // pair-bias heads: out_bias[h][q][k] with (q, k) the pixel's own (row, col)
  for (int h0 = 0; h0 < a.n_bias; h0 += 32) {
    load_w_rows(a.w_bias + (int64_t)h0 * C, sW, 32, tid);  // host pads w_bias to a multiple of 32 rows
    lds_barrier();
    f32x16 acc[1];
    mfma_chunk<true, 1>(xf, sW, lane, acc);
    const int p = wave * 32 + (lane & 31);
    if (t.valid(p)) {
      const int64_t pixel = t.pix(p);  // = q * N + k
      const int q = (int)(pixel / a.N), k = (int)(pixel % a.N);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int h = h0 + acc_row(r, lane);
        if (h < a.n_bias) {
          if (a.out_bias_bf16)
            a.out_bias_bf16[((int64_t)h * a.N + q) * a.ld_bias + k] = f2bf(acc[0][r] * a.bias_scale);
          else
            a.out_bias[(int64_t)h * a.N * a.N + pixel] = acc[0][r];
        }
      }
    }
    lds_barrier();
  }
}

// ============================================================================
// triangle attention: output gate and output projection
// ============================================================================
// The attention core leaves the normalised, ungated output.  The gate sigmoid(LN(x) Wg^T) belongs to the
// same pixel of the pair tensor that this kernel reads anyway for the residual, so it is computed here
// (one LayerNorm and one 128 x 128 product per pixel) instead of making a round trip through memory as a
// fourth projection plane.  The gate comes out of its MFMAs in T form (a lane owns a pixel and, per
// register quad, 4 consecutive weight rows); with the weight rows permuted on their way into LDS (row rho
// holds channel swap23(rho): bits 2 and 3 exchanged) a lane-half's registers 8 a .. 8 a + 7 of tile nt are
// the eight consecutive channels 32 nt + 16 a + 8 hh .. of its pixel: exactly the B fragment of k-step
// 2 nt + a of the output projection, so gate and attention output meet register by register.
template <typename TIO>
__global__ __launch_bounds__(256, 2) void attn_out_kernel(AttnOutArgs a) {
  __shared__ __attribute__((aligned(16))) bf16_t smem[2 * TM * LDX];
  bf16_t* sX = smem;
  bf16_t* sW = smem + TM * LDX;
  float* sS = reinterpret_cast<float*>(smem);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const Tile t = make_tile(a.N, a.transpose != 0);  // where the result lands in the pair tensor
  // Loads are unconditional (rows past the end re-read a valid one and are zeroed / skipped later).
  // The attention output is requested once the gate's MFMAs are issued (its 32 registers would not
  // fit beside them), and the pair rows are read a second time, out of the cache, for the residual:
  // keeping them in registers from the LayerNorm on costs more (spills, or a bf16-rounded gate)
  // than the second read (measured).
  const TIO* x = reinterpret_cast<const TIO*>(a.pair);
  const int ck = tid & 15, prow = tid >> 4;
  WChunkRegs wr;
  wr.load<true>(a.w_gate, tid);
  load_ln_tile<TIO>(x, t, a.ln_w, a.ln_b, sX, tid, a.skip_ln != 0, a.lw.inv_c, a.lw.pad);
  wr.store(sW, tid);
  lds_barrier();
  bf16x8 xf[8];
  load_x_frags(sX, wave, lane, xf);
  f32x16 gate[4];
  mfma_chunk<true, 4>(xf, sW, lane, gate);
  // the attention output and the output weights travel while the sigmoids are taken
  u32x4 og[8];
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int p = it * 16 + prow;
    og[it] = *reinterpret_cast<const u32x4*>(a.og + ((int64_t)t.o * a.N + t.r0 + (t.valid(p) ? p : 0)) * a.ld_og + ck * 8);
  }
  wr.load<false>(a.w_out, tid);
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int r = 0; r < 16; ++r) gate[nt][r] = sigmoidf_(gate[nt][r]);
  lds_barrier();  // every wave is done with the LayerNorm tile and the gate weights
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int p = it * 16 + prow;
    const u32x4 z = {0, 0, 0, 0};
    *reinterpret_cast<u32x4*>(sX + p * LDX + ck * 8) = t.valid(p) ? og[it] : z;
  }
  wr.store(sW, tid);
  lds_barrier();
  load_x_frags(sX, wave, lane, xf);
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    float f[8];
    unpack8(__builtin_bit_cast(u32x4, xf[ks]), f);
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] *= gate[ks >> 1][8 * (ks & 1) + e];
    xf[ks] = as_frag(pack8(f));
  }
  f32x16 acc[4];
  mfma_chunk<true, 4>(xf, sW, lane, acc);
  lds_barrier();
  stage_t_f32(acc, sS, wave, lane);
  lds_barrier();
  store_tile_f32<TIO>(sS, t, reinterpret_cast<TIO*>(a.out), a.residual ? x : nullptr, tid);
}

// ============================================================================
// SwiGLU transition, c = 128, hidden = 128 * factor, all in one kernel
// ============================================================================
// Weight slabs go from global memory straight into LDS (global_load_lds_dwordx4: no staging
// registers, no LDS stores in the instruction stream).  Such a load puts lane l's 16 bytes at
// base + 16 l, so rows cannot be padded; their 16-byte chunks are XOR-permuted instead, on the
// global side, where a lane is free to fetch any chunk.
template <int OFF>
__device__ __forceinline__ void lds_dma16(const char* gbase, uint32_t voff, const char* dst) {
  const uint32_t lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)dst;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3"
               :: "s"(lds), "v"(voff), "s"(gbase), "n"(OFF) : "memory", "m0");
}
// workgroup barrier that also waits for this wave's loads into LDS
__device__ __forceinline__ void dma_lds_barrier() {
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

constexpr int W1_SLAB = 64 * 256;  // 32 "a" rows + 32 "b" rows of 128 bf16: 16 KB
constexpr int W2_SLAB = 128 * 64;  // 128 output rows x 32 hidden units: 8 KB

template <typename TIO>
__global__ __launch_bounds__(256, 2) void transition_kernel(TransitionArgs a) {
  // The hidden layer is walked in slabs of 32 units.  Per slab a wave issues 16 MFMAs of GEMM1 (T form:
  // a^T and b^T, 32 hidden x 32 pixels each), 32 SiLU-gate evaluations per lane pair of registers and 8
  // MFMAs of GEMM2 into the four output tiles; h^T = silu(a) * b in registers 8s..8s+7 is, as it stands,
  // the B fragment of k-step s of GEMM2 when row rho of the slab holds hidden unit swap23(rho) (bits 2
  // and 3 exchanged): the lane-half's eight registers are then eight consecutive units, one 16-byte
  // fragment of W2's natural order.
  //
  // The slabs run as a software pipeline inside each wave: the MFMAs of GEMM1 of slab h are issued one by
  // one with the gating of slab h - 1 between them, and the MFMAs of GEMM2 of slab h - 1 follow as their
  // fragments become complete.  Phases run back to back would cost the sum of the matrix unit's and the
  // vector unit's time (the two do not overlap between the waves of a SIMD).  W1 slabs are double-
  // buffered, W2 slabs triple-buffered (a W2 slab is used one iteration after its W1 slab); one barrier
  // per slab.
  __shared__ __attribute__((aligned(1024))) char smem[2 * TM * LDX * 2];  // 69.6 KB
  // layout: [0, 34816) LN tile, later W1 buffer 1 (16 KB) and W2 buffers 1, 2 (8 KB each);
  //         [34816, 34816 + 24 KB) W1 buffer 0 and W2 buffer 0, loaded while the LN tile is being made
  static_assert(TM * LDX * 2 >= W1_SLAB + 2 * W2_SLAB, "buffers 1, 2 fit the LN tile");
  static_assert(TM * LDX * 2 + W1_SLAB + W2_SLAB <= (int)sizeof(smem), "buffers 0 fit behind it");
  static_assert(TM * LDS_F * 4 <= (int)sizeof(smem), "staging tile must fit");
  bf16_t* sX = reinterpret_cast<bf16_t*>(smem);
  float* sS = reinterpret_cast<float*>(smem);
  char* const w1buf0 = smem + TM * LDX * 2;
  char* const w1buf1 = smem;
  char* const w2buf0 = smem + TM * LDX * 2 + W1_SLAB;
  char* const w2buf1 = smem + W1_SLAB;
  char* const w2buf2 = smem + W1_SLAB + W2_SLAB;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j = lane & 31, hh = lane >> 5;
  const Tile t = make_tile(a.N, false);
  const TIO* x = reinterpret_cast<const TIO*>(a.x);
  const int n_slabs = a.hidden / 32;

  // ---- loads into LDS: per-lane global offsets, wave-uniform LDS destinations ----
  // W1 slab h: rows of the host-packed [hidden/64][64 a | 64 b][128] array; LDS row rho (0..31 a, 32..63 b)
  // holds unit swap23(rho % 32); chunk c of a row at position c ^ (rho & 15).  Load i of 4 covers rows
  // 16 i + lane / 16 (of this wave's quarter: rows 16 i + 4 wave + ...), one 16-byte chunk per lane.
  const char* w1g = reinterpret_cast<const char*>(a.w1);
  const char* w2g = reinterpret_cast<const char*>(a.w2);
  uint32_t w1off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int rho = 16 * i + 4 * wave + (lane >> 4);              // 0..63
    const int u = rho & 31;
    const int unit = (u & ~12) | ((u & 4) << 1) | ((u & 8) >> 1);  // swap23
    const int chunk = (lane & 15) ^ (rho & 15);
    w1off[i] = (uint32_t)((((rho >> 5) * 64 + unit) * C + chunk * 8) * 2);  // + slab base (below)
  }
  // W2 slab h: rows o = 0..127 of w2[128][hidden], columns 32 h .. + 31 (four 16-byte chunks); chunk c of
  // row o at position c ^ ((o >> 2) & 3).  Load i of 2 covers rows 64 i + 16 wave + lane / 4.
  uint32_t w2off[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int o = 64 * i + 16 * wave + (lane >> 2);
    const int chunk = (lane & 3) ^ ((o >> 2) & 3);
    w2off[i] = (uint32_t)((o * a.hidden + chunk * 8) * 2);
  }
  auto load_slab = [&](int h, char* w1dst, char* w2dst) {
    // slab h = half (h & 1) of the 64-unit block h / 2: a rows 32 (h & 1) .., b rows 64 + 32 (h & 1) ..
    const uint32_t base1 = (uint32_t)(((h >> 1) * 128 + (h & 1) * 32) * C * 2);
    const uint32_t base2 = (uint32_t)(h * 32 * 2);
#pragma unroll
    for (int i = 0; i < 4; ++i) lds_dma16<0>(w1g, w1off[i] + base1, w1dst + (16 * i + 4 * wave) * 256);
#pragma unroll
    for (int i = 0; i < 2; ++i) lds_dma16<0>(w2g, w2off[i] + base2, w2dst + (64 * i + 16 * wave) * 64);
  };
  load_slab(0, w1buf0, w2buf0);

  load_ln_tile<TIO>(x, t, a.ln_w, a.ln_b, sX, tid, false, a.lw.inv_c, a.lw.pad);
  lds_barrier();
  bf16x8 xf[8];
  load_x_frags(sX, wave, lane, xf);
  dma_lds_barrier();  // sX is free from here on; slab 0 has landed
  if (n_slabs > 1) load_slab(1, w1buf1, w2buf1);

  f32x16 out[4], zero16;
#pragma unroll
  for (int r = 0; r < 16; ++r) zero16[r] = 0.f;
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) out[nt] = zero16;

  // fragment addresses: W1 row (32 tile + j), chunk 2 ks + hh; W2 row (32 ot + j), chunk 2 s + hh
  const int w1frag = j * 256, w1sw = j & 15;
  const int w2frag = j * 64, w2sw = (j >> 2) & 3;
  auto w1_frag = [&](const char* buf, int tile, int ks) {
    return as_frag(*reinterpret_cast<const u32x4*>(buf + tile * (32 * 256) + w1frag + (((2 * ks + hh) ^ w1sw) << 4)));
  };
  auto w2_frag = [&](const char* buf, int ot, int s) {
    return as_frag(*reinterpret_cast<const u32x4*>(buf + ot * (32 * 64) + w2frag + (((2 * s + hh) ^ w2sw) << 4)));
  };

  f32x16 abA[2], abB[2];  // [0] a^T, [1] b^T of a slab; A: even slabs, B: odd slabs
  // One iteration: GEMM1 of slab h into `cur` (h < n_slabs) out of W1 buffer `w1`; gating of slab h - 1 out
  // of `prev` and its GEMM2 out of W2 buffer `w2p` (h > 0).
  // (the second k-step of a slab's GEMM2 is issued behind the first groups of the NEXT iteration: its
  // fragments are complete only when the last group of this one is through)
  bf16x8 w2f[4];
  u32x4 hfrag[2];
  auto iteration = [&](auto g1_c, auto g2_c, auto carry_c, const char* w1, const char* w2p, f32x16* cur, f32x16* prev) {
    constexpr bool gemm1 = decltype(g1_c)::value, gemm2 = decltype(g2_c)::value, carry = decltype(carry_c)::value;
    bf16x8 wf[3];
    if (gemm1) {
      wf[0] = w1_frag(w1, 0, 0);
      wf[1] = w1_frag(w1, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < 16; ++m) {
      // GEMM2, k-step 1 of the slab gated in the previous iteration
      if (carry && m < 4) out[m] = mfma32(w2f[m], as_frag(hfrag[1]), out[m]);
      // MFMA m of GEMM1: k-step m / 2, tile m % 2 (a, b)
      if (gemm1) {
        if (m + 2 < 16) wf[(m + 2) % 3] = w1_frag(w1, (m + 2) & 1, (m + 2) >> 1);
        cur[m & 1] = mfma32(wf[m % 3], xf[m >> 1], m < 2 ? zero16 : cur[m & 1]);
      }
      if (gemm2) {
        // register m of the previous slab: h = silu(a) * b
        const float av = prev[0][m], bv = prev[1][m];
        float hv = av * sigmoidf_(av) * bv;
        asm volatile("" : "+v"(hv));  // keeps the arithmetic in this group
        prev[0][m] = hv;
        if (m == 3 || m == 12) {
          // the W2 fragments of k-step 0 (used behind groups 8..11) and, once those are through, of k-step 1
#pragma unroll
          for (int ot = 0; ot < 4; ++ot) w2f[ot] = w2_frag(w2p, ot, m == 3 ? 0 : 1);
        }
        if ((m & 7) == 7) {
          const int s8 = m & 8;
          float f8[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) f8[e] = prev[0][s8 + e];
          hfrag[m >> 3] = pack8(f8);
        }
        // GEMM2 of k-step 0 behind groups 8..11
        if (m >= 8 && m < 12) out[m - 8] = mfma32(w2f[m - 8], as_frag(hfrag[0]), out[m - 8]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // slab h: W1 buffer h % 2, W2 buffer h % 3; the loads of slab h + 1 are issued at the top of iteration h
  // (its W1 buffer was last read in iteration h - 1, its W2 buffer in iteration h - 1 as slab h - 2's)
  using T_ = std::true_type;
  using F_ = std::false_type;
  auto w2buf = [&](int h) -> char* { return h % 3 == 0 ? w2buf0 : (h % 3 == 1 ? w2buf1 : w2buf2); };
  // slab 0: GEMM1 only
  iteration(T_{}, F_{}, F_{}, w1buf0, w2buf0, abA, abB);
  dma_lds_barrier();
  // slab 1 (gating of slab 0: nothing carried over yet)
  if (n_slabs > 2) load_slab(2, w1buf0, w2buf(2));
  iteration(T_{}, T_{}, F_{}, w1buf1, w2buf(0), abB, abA);
  dma_lds_barrier();
#pragma unroll 1
  for (int h = 2; h < n_slabs; h += 2) {
    // even slab h, then odd slab h + 1 (n_slabs is even)
    load_slab(h + 1, w1buf1, w2buf(h + 1));
    iteration(T_{}, T_{}, T_{}, w1buf0, w2buf(h - 1), abA, abB);
    dma_lds_barrier();
    if (h + 2 < n_slabs) load_slab(h + 2, w1buf0, w2buf(h + 2));
    iteration(T_{}, T_{}, T_{}, w1buf1, w2buf(h), abB, abA);
    dma_lds_barrier();
  }
  // gating and GEMM2 of the last slab (odd: in abB), then its second k-step
  iteration(F_{}, T_{}, T_{}, w1buf0, w2buf(n_slabs - 1), abA, abB);
#pragma unroll
  for (int ot = 0; ot < 4; ++ot) out[ot] = mfma32(w2f[ot], as_frag(hfrag[1]), out[ot]);
  dma_lds_barrier();
  stage_t_f32(out, sS, wave, lane);
  lds_barrier();
  store_tile_f32<TIO>(sS, t, reinterpret_cast<TIO*>(a.out), a.residual ? x : nullptr, tid);
}

// ============================================================================
// diffusion conditioning: pair_cond = Linear(LayerNorm([pair | relative encoding]))
// ============================================================================
// The 267 input channels of a pixel (i, j) are the 128 pair channels and 139 one-hot channels of the
// relative encoding: clipped residue offset inside a chain (2r + 2 classes), clipped token offset inside a
// residue (2r + 2), same entity (1), clipped chain-copy offset inside an entity (2c + 2); r = 32, c = 2.
// The concatenated tensor is never made.  A pixel holds n1 = 3 + same_entity ones, so its LayerNorm
// statistics are mean = (sum x + n1) / 267, E[x^2] = (sum x^2 + n1) / 267, and with the weight rows of the
// one-hot channels h folded with their LayerNorm weights, G[h][o] = ln_w[h] W[o][h],
//   out[o] = sum_{c < 128} LN(x)_c W[o][c]  +  rstd * (sum_{hot h} G[h][o]  -  mean * sum_h G[h][o]).
// The first term is the tile product of the other kernels here (LayerNorm-ed pixels as bf16 fragments);
// the second is four rows of a 139 x 128 fp32 table per pixel, added in fp32.
template <typename TIO>
__global__ __launch_bounds__(256, 2) void pair_cond_init_kernel(PairCondInitArgs a) {
  __shared__ __attribute__((aligned(16))) bf16_t smem[2 * TM * LDX];
  bf16_t* sX = smem;
  bf16_t* sW = smem + TM * LDX;
  float* sS = reinterpret_cast<float*>(smem);
  __shared__ float sRstd[TM], sMeanRstd[TM];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const Tile t = make_tile(a.N, false);
  const TIO* x = reinterpret_cast<const TIO*>(a.pair);
  using E = Elem<TIO>;
  constexpr int NB = E::kBatch;
  const int chunk = tid & 15, prow = tid >> 4;
  const int i = t.o;
  const int ent_i = a.entity_id[i];
  const float inv_c = 1.f / (float)(C + a.n_rel);

  WChunkRegs wr;
  wr.load(a.w_pair, tid);
  float w[8];
  load_param8(a.ln_w + chunk * 8, 1.f, w);
#pragma unroll
  for (int base = 0; base < 8; base += NB) {
    typename E::Raw raw[NB];
    int ent_j[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int p = (base + b) * 16 + prow;
      const int pc = t.valid(p) ? p : 0;
      raw[b] = E::load_raw(x + t.pix(pc) * C + chunk * 8);
      ent_j[b] = a.entity_id[t.r0 + pc];
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int p = (base + b) * 16 + prow;
      float v[8], o[8];
      E::unpack_raw(raw[b], v);
      float s = 0.f, q = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) { v[e] *= a.in_scale; s += v[e]; q = fmaf(v[e], v[e], q); }
      const float n1 = 3.f + (ent_j[b] == ent_i ? 1.f : 0.f);
      const float mean = (group16_sum(s) + n1) * inv_c;
      const float var = fmaxf(fmaf(group16_sum(q) + n1, inv_c, -mean * mean), 0.f);
      const float rstd = rsqrtf(var + LN_EPS);
      const float shift = -mean * rstd;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = fmaf(v[e], rstd, shift) * w[e];
      u32x4 pk = pack8(o);
      if (!t.valid(p)) pk = u32x4{0u, 0u, 0u, 0u};
      *reinterpret_cast<u32x4*>(sX + p * LDX + chunk * 8) = pk;
      if (chunk == 0) { sRstd[p] = rstd; sMeanRstd[p] = mean * rstd; }
    }
  }
  wr.store(sW, tid);
  lds_barrier();
  bf16x8 xf[8];
  load_x_frags(sX, wave, lane, xf);
  f32x16 acc[4];
  mfma_chunk<true, 4>(xf, sW, lane, acc);

  // the lane's pixel: its four hot rows of the table
  const int px = wave * 32 + (lane & 31), hh = lane >> 5;
  const int j = t.r0 + (t.valid(px) ? px : 0);
  const int r = a.max_rel_idx, c2 = a.max_rel_chain;
  const bool same_chain = a.asym_id[i] == a.asym_id[j];
  const int dres = a.residue_index[i] - a.residue_index[j];
  const int h_res = same_chain ? min(max(dres + r, 0), 2 * r) : 2 * r + 1;
  const int h_tok = (same_chain && dres == 0) ? min(max(a.token_index[i] - a.token_index[j] + r, 0), 2 * r) : 2 * r + 1;
  const bool same_ent = a.entity_id[j] == ent_i;
  const int h_sym = same_ent ? min(max(a.sym_id[i] - a.sym_id[j] + c2, 0), 2 * c2) : 2 * c2 + 1;
  const float* g0 = a.g_hot + (int64_t)h_res * C;
  const float* g1 = a.g_hot + (int64_t)(2 * r + 2 + h_tok) * C;
  const float* g2 = a.g_hot + (int64_t)(4 * r + 4) * C;              // same entity
  const float* g3 = a.g_hot + (int64_t)(4 * r + 5 + h_sym) * C;
  const float ent_f = same_ent ? 1.f : 0.f;
  const float rstd = sRstd[px], mrstd = sMeanRstd[px];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int ch = nt * 32 + 8 * g + 4 * hh;
      const f32x4 v0 = *reinterpret_cast<const f32x4*>(g0 + ch), v1 = *reinterpret_cast<const f32x4*>(g1 + ch);
      const f32x4 v2 = *reinterpret_cast<const f32x4*>(g2 + ch), v3 = *reinterpret_cast<const f32x4*>(g3 + ch);
      const f32x4 so = *reinterpret_cast<const f32x4*>(a.g_sum + ch);
      const float hot[4] = {v0.x + v1.x + ent_f * v2.x + v3.x, v0.y + v1.y + ent_f * v2.y + v3.y,
                            v0.z + v1.z + ent_f * v2.z + v3.z, v0.w + v1.w + ent_f * v2.w + v3.w};
      const float sum[4] = {so.x, so.y, so.z, so.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[nt][4 * g + e] += rstd * hot[e] - mrstd * sum[e];
    }
  lds_barrier();
  stage_t_f32(acc, sS, wave, lane);
  lds_barrier();
  store_tile_f32<float>(sS, t, a.out, nullptr, tid);
}

template <typename K, typename A>
int launch_tiles(K kern, const A& a, int64_t n_outer, int N, hipStream_t stream) {
  const int64_t tiles = n_outer * ((N + TM - 1) / TM);
  if (tiles <= 0 || tiles > 0x7fffffff) return AF3_ERR_BAD_ARG;
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(256), 0, stream, a);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

int launch_trimul_prologue(const TriMulArgs& a, hipStream_t s) {
  if (a.N <= 0 || a.Np < a.N || (a.Np & 7) || !a.pair || !a.a_buf || !a.b_buf || !a.w_pg) return AF3_ERR_BAD_ARG;
  if (!aligned16(a.pair) || !aligned16(a.a_buf) || !aligned16(a.b_buf) || !aligned16(a.w_pg)) return AF3_ERR_BAD_ARG;
  return a.io_f32 ? launch_tiles(trimul_prologue_kernel<float>, a, a.N, a.N, s)
                  : launch_tiles(trimul_prologue_kernel<bf16_t>, a, a.N, a.N, s);
}
int launch_trimul_epilogue(const TriMulArgs& a, hipStream_t s) {
  if (a.N <= 0 || a.Np < a.N || (a.Np & 7) || !a.pair || !a.t_buf || !a.out || !a.w_gl || !a.w_out ||
      !a.ln_c_w || !a.ln_c_b)
    return AF3_ERR_BAD_ARG;
  if (!aligned16(a.pair) || !aligned16(a.t_buf) || !aligned16(a.out) || !aligned16(a.w_gl) || !aligned16(a.w_out))
    return AF3_ERR_BAD_ARG;
  return a.io_f32 ? launch_tiles(trimul_epilogue_kernel<float>, a, a.N, a.N, s)
                  : launch_tiles(trimul_epilogue_kernel<bf16_t>, a, a.N, a.N, s);
}
int launch_attn_proj(const AttnProjArgs& a, hipStream_t s) {
  if (a.N <= 0 || !a.pair || a.n_chunks < 0 || a.n_chunks > 4 || a.n_bias < 0) return AF3_ERR_BAD_ARG;
  if (a.n_chunks > 0 && (!a.w_main || !a.out_main || (a.ld_main & 7) || a.ld_main < a.n_chunks * C)) return AF3_ERR_BAD_ARG;
  if (a.n_bias > 0 && (!a.w_bias || (!a.out_bias && !a.out_bias_bf16))) return AF3_ERR_BAD_ARG;
  if (a.out_bias_bf16 && a.ld_bias < a.N) return AF3_ERR_BAD_ARG;
  if (!aligned16(a.pair) || !aligned16(a.w_main) || !aligned16(a.out_main) || !aligned16(a.w_bias)) return AF3_ERR_BAD_ARG;
  return a.io_f32 ? launch_tiles(attn_proj_kernel<float>, a, a.N, a.N, s)
                  : launch_tiles(attn_proj_kernel<bf16_t>, a, a.N, a.N, s);
}
int launch_attn_out(const AttnOutArgs& a, hipStream_t s) {
  if (a.N <= 0 || !a.og || !a.w_out || !a.w_gate || !a.out || (a.ld_og & 7) || !a.pair) return AF3_ERR_BAD_ARG;
  if ((a.ln_w == nullptr) != (a.ln_b == nullptr) || (a.skip_ln == 0) != (a.ln_w != nullptr)) return AF3_ERR_BAD_ARG;
  if (!aligned16(a.og) || !aligned16(a.w_out) || !aligned16(a.w_gate) || !aligned16(a.out) || !aligned16(a.pair))
    return AF3_ERR_BAD_ARG;
  return a.io_f32 ? launch_tiles(attn_out_kernel<float>, a, a.N, a.N, s)
                  : launch_tiles(attn_out_kernel<bf16_t>, a, a.N, a.N, s);
}
int launch_pair_cond_init(const PairCondInitArgs& a, hipStream_t s) {
  if (a.N <= 0 || !a.pair || !a.out || !a.w_pair || !a.ln_w || !a.g_hot || !a.g_sum || !a.asym_id || !a.residue_index ||
      !a.token_index || !a.entity_id || !a.sym_id)
    return AF3_ERR_BAD_ARG;
  if (a.max_rel_idx < 0 || a.max_rel_chain < 0 || a.n_rel != 4 * a.max_rel_idx + 2 * a.max_rel_chain + 7) return AF3_ERR_BAD_ARG;
  if (!aligned16(a.pair) || !aligned16(a.out) || !aligned16(a.w_pair) || !aligned16(a.g_hot) || !aligned16(a.g_sum) ||
      !aligned16(a.ln_w))
    return AF3_ERR_BAD_ARG;
  return a.io_f32 ? launch_tiles(pair_cond_init_kernel<float>, a, a.N, a.N, s)
                  : launch_tiles(pair_cond_init_kernel<bf16_t>, a, a.N, a.N, s);
}
int launch_transition(const TransitionArgs& a, hipStream_t s) {
  // x is [rows][128]; handled as `rows` positions in one long row
  if (a.N <= 0 || !a.x || !a.out || !a.w1 || !a.w2 || a.hidden <= 0 || (a.hidden & 63)) return AF3_ERR_BAD_ARG;
  if (!aligned16(a.x) || !aligned16(a.out) || !aligned16(a.w1) || !aligned16(a.w2)) return AF3_ERR_BAD_ARG;
  return a.io_f32 ? launch_tiles(transition_kernel<float>, a, 1, a.N, s)
                  : launch_tiles(transition_kernel<bf16_t>, a, 1, a.N, s);
}
