// Triangle attention, the fast path: projection kernel + flash kernel that
// share a head-major scratch layout.
//
// Scratch layout (bf16), for rows b of the (possibly transposed) operator:
//   Q, K, G : [b][h][s][32]          one 4 KB-contiguous slab per 64 positions
//   Vt      : [b][h][32][ldn]        V transposed (keys contiguous), ldn = N up to 8
//   bias    : MFMA-fragment order     pair bias * log2(e) (tri_bias_offset); keys >= N zero
// so every tile the flash kernel stages is a run of full 16-byte chunks with no
// transposition and no boundary code.
//
// Flash kernel: same wave-level scheme as attention.hip (S^T = K Q^T so a lane
// owns one query; bf16 probabilities feed O^T += V^T P^T directly), plus
//   * exponentials in base 2 (log2(e) folded into q and the bias upstream);
//   * the pair bias is the INITIAL VALUE of the MFMA accumulator;
//   * the key mask rides in the matrix product: K gets a 33rd column holding 0,
//     -1e9 (masked key) or -inf (tile padding) and Q a matching 1.0.  A masked
//     logit is bias + q.k - 1e9, which fp32 rounds to -1e9 for every key alike:
//     masked keys get weight exactly 0 and a fully masked row is uniform, as
//     with the reference's additive 1e9 * (mask - 1);
//   * workgroup ids are remapped so that each XCD (ids are dealt round-robin to
//     the 8 XCDs) walks a contiguous range of (head, row, query-tile): the six
//     query tiles that share one row's K/V, and the head's bias, stay in that
//     XCD's L2.
#include "common.h"
#include "kernels.h"
#include <type_traits>

#include "tile_common.h"

namespace {

constexpr int H = 4, D = 32;

// ============================================================================
// projections: LN -> q (scaled), k, sigmoid gate (position-major) and v
// (channel-major), + pair-bias heads
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
  // Step s = 2 * chunk + half: weight rows 64 half .. + 63 of chunk s / 2 (chunks q, k, v, g as packed in
  // w_qkvg), four 16-byte pieces per thread; the 32 (padded) pair-bias rows ride in the same registers.
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
  load_ln_tile<TIO>(x, t, a.ln_w, a.ln_b, sX, tid, a.skip_ln != 0);
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
    if (step < 7) wload(step + 1);
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
            *reinterpret_cast<u32x2*>(sX + ch * LDX + p0) = pk;
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
              v[e] = chunk == 0 ? y * a.q_scale : (chunk == 3 ? sigmoidf_(y) : y);
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
    if (step < 7) wstore(4);
    else if (a.n_bias > 0) wstore(2);
    if (pairt == 1) {
      // both halves of the chunk are staged: 128 channels per position go out
      if (chunk == 2) {
        // Vt[(b*H + h)*32 + d][s]: per channel 128 consecutive positions
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int idx = tid + 256 * i, ch = idx >> 4, pc = idx & 15;
          const int r = t.r0 + pc * 8;
          if (r < a.ldn)
            *reinterpret_cast<u32x4*>(a.vt + (bh0 * D + ch) * a.ldn + r) =
                *reinterpret_cast<const u32x4*>(sX + ch * LDX + pc * 8);
        }
      } else {
        bf16_t* plane = chunk == 0 ? a.q : (chunk == 1 ? a.k : a.g);
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
  do_step(std::integral_constant<int, 6>{});
  do_step(std::integral_constant<int, 7>{});

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
            a.bias[tri_bias_offset(a.N, h, t.o, r)] = f2bf(t.valid(p) ? acc[0][h] * a.bias_scale : 0.f);
        }
      } else if (t.valid(p)) {
        // q = r, k = o
#pragma unroll
        for (int h = 0; h < H; ++h) {
          a.bias[tri_bias_offset(a.N, h, r, t.o)] = f2bf(acc[0][h] * a.bias_scale);
          if (t.o == a.N - 1)
            for (int k = a.N; k < kpad; ++k) a.bias[tri_bias_offset(a.N, h, r, k)] = 0;
        }
      }
    }
  }
}

// ============================================================================
// flash attention core
// ============================================================================
constexpr int KT = 64;       // keys per LDS tile
constexpr int LDK = 56;      // sK row: 32 head-dim + 16 mask k-step + 8 pad (bf16); 112 B
constexpr int LDV = KT + 4;  // sVt row: 136 B = 34 dwords, so 32 lanes' 8-byte reads hit 32 bank pairs
constexpr int QW = 128;      // queries per workgroup
constexpr uint32_t BF16_ONE = 0x3F80u, BF16_NEG_INF = 0xFF80u, BF16_NEG_1E9 = 0xCE6Eu;

// One workgroup = (row b, head h, 128 queries); a wave owns 32 queries, lane
// (j, hh) holds query j's scores for half of the keys of each 32-key tile.
//
// S^T = K Q^T runs on the matrix unit with three k-steps: the two halves of the
// head dimension and a mask step (K column 32 = 0, -1e9 or -inf per key, times a
// Q entry of 1.0).  The pair bias is added on the matrix unit too,
// S^T += I * bias^T; its B fragments are 16 contiguous bytes per lane and come
// straight from global memory, where the bias is stored in fragment order: each
// load instruction covers one contiguous 1 KB run (the bias is shared by every
// row b and stays L2-resident), fetched one tile ahead.  Only K and V^T go
// through LDS, double-buffered (23 KB), with one barrier per tile; three
// workgroups fit on a CU, and with head dim 32 it is the number of waves
// available to hide the MFMA -> softmax -> MFMA dependency chain that sets the pace.
template <bool HAS_BIAS>
__global__ __launch_bounds__(256, 3) void triattn_flash_kernel(TriAttnArgs a) {
  __shared__ __attribute__((aligned(16))) bf16_t sK[2][KT * LDK];
  __shared__ __attribute__((aligned(16))) bf16_t sVt[2][D * LDV];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hh = lane >> 5, j = lane & 31;
  const int xaddr = half_swap_addr();
  const int N = a.N;
  const int QT = (N + QW - 1) / QW;
  // Workgroup ids are dealt round-robin to the 8 XCDs.  The query tiles of one
  // (row, head) share its K / V and run back to back on one XCD (id = slot * 8 +
  // xcd, query tile fastest within the XCD's slots); the (row, head) pairs
  // themselves are dealt to the XCDs in turn, rows ascending, so that the whole
  // chip moves through the rows together, starting with the ones the
  // projection kernel wrote last.
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int qt = slot % QT;
  const int pair_idx = (slot / QT) * 8 + xcd;
  if (pair_idx >= H * N) return;
  const int b = pair_idx / H;
  const int h = pair_idx % H;
  const int q0 = qt * QW;
  const int qw = q0 + wave * 32 + j;
  const int qi = min(qw, N - 1);
  const int64_t bh = (int64_t)b * H + h;
  const int ldn = (int)a.ldn;

  bf16x8 qf[3];
  {
    const bf16_t* qp = a.q + (bh * N + qi) * D + 8 * hh;
    qf[0] = as_frag(*reinterpret_cast<const u32x4*>(qp));
    qf[1] = as_frag(*reinterpret_cast<const u32x4*>(qp + 16));
    u32x4 one = {hh == 0 ? BF16_ONE : 0u, 0u, 0u, 0u};
    qf[2] = as_frag(one);
  }
  // Identity fragments: A-fragment of k-step `st`: lane (row i = j, half hh)
  // holds I[i][16 st + 8 hh + e], e = 0..7: a single 1.0 where 16 st + 8 hh + e == i.
  bf16x8 idf[2];
#pragma unroll
  for (int st = 0; st < 2; ++st) {
    const int e1 = j - 16 * st - 8 * hh;
    uint32_t w[4] = {0u, 0u, 0u, 0u};
    if (e1 >= 0 && e1 < 8) w[e1 >> 1] = (e1 & 1) ? (BF16_ONE << 16) : BF16_ONE;
    idf[st] = as_frag(u32x4{w[0], w[1], w[2], w[3]});
  }

  const bf16x8 onesf = as_frag(u32x4{0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u});

  // LDS loaders, one 16-byte chunk each per tile:
  //   K   thread (key = tid / 4, c = tid % 4)   + the mask k-step by c < 2
  //   Vt  thread (d = tid / 8, kc = tid % 8)
  const int k_key = tid >> 2, k_c = tid & 3;
  const int v_d = tid >> 3, c8 = (tid & 7) * 8;
  // All global loads are unconditional, from clamped addresses, and nothing is
  // decided from a loaded value until the LDS store one tile later: a load
  // under a lane mask, or a value inspected right after its load, would put a
  // full memory round trip (behind every load queued before it) into each tile.
  // Addresses are a wave-uniform 64-bit base plus a 32-bit lane offset.
  u32x4 rk, rv, rb[4];  // rb: bias fragments, fetched one tile ahead
  float rm = 1.f;
  bool key_ok = false, col_ok = false;
  const char* kbase = reinterpret_cast<const char*>(a.k + bh * N * D);
  const char* vbase = reinterpret_cast<const char*>(a.vt + bh * D * a.ldn);
  const char* mbase = reinterpret_cast<const char*>(a.mask ? a.mask + (int64_t)b * N : nullptr);
  const uint32_t v_row = (uint32_t)(v_d * ldn) * 2u;
  auto gload_kv = [&](int k0) {
    key_ok = k0 + k_key < N;
    col_ok = k0 + c8 < ldn;
    const uint32_t key = (uint32_t)min(k0 + k_key, N - 1);
    rk = *reinterpret_cast<const u32x4*>(kbase + (key * (D * 2u) + k_c * 16u));
    if (mbase) rm = *reinterpret_cast<const float*>(mbase + key * 4u);
    rv = *reinterpret_cast<const u32x4*>(vbase + (v_row + (col_ok ? (uint32_t)(k0 + c8) * 2u : 0u)));
  };
  // bias B-fragment i = 2 u + st of a tile: keys 32 u + 16 st + 8 hh .. + 8 of this
  // lane's query.  A query beyond N reads its (uninitialised) slot of the padded
  // block, or block 0 if its whole block lies beyond N; whatever it reads only
  // reaches its own, discarded, column of S.
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int qblock = q0 + wave_u * 32 < N ? (q0 >> 5) + wave_u : 0;
  const char* bbase = HAS_BIAS ? reinterpret_cast<const char*>(a.bias + tri_bias_offset(N, h, qblock * 32, 0)) : nullptr;
  const uint32_t b_lane = (uint32_t)(j * 16 + 8 * hh) * 2u;
  const int bias_tiles = (int)tri_bias_ktiles(N);
  auto gload_bias = [&](u32x4* dst, int tile) {  // a tile past the end re-reads the last one
    if (!HAS_BIAS) return;
    const char* p = bbase + (size_t)min(tile, bias_tiles - 1) * 4096u;
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[i] = *reinterpret_cast<const u32x4*>(p + (b_lane + 1024u * i));
  };
  // A key at or past N gets -inf in its mask entry, so its probability is
  // exactly zero whatever its K row and V column hold; the clamped loads gave
  // them finite values (the last row / the first chunk), which is all it takes.
  auto sstore = [&](int buf) {
    *reinterpret_cast<u32x4*>(&sK[buf][k_key * LDK + k_c * 8]) = rk;
    if (k_c < 2) {
      const uint32_t rmask = !key_ok ? BF16_NEG_INF : (rm == 0.f ? BF16_NEG_1E9 : 0u);
      u32x4 m = {k_c == 0 ? rmask : 0u, 0u, 0u, 0u};
      *reinterpret_cast<u32x4*>(&sK[buf][k_key * LDK + 32 + k_c * 8]) = m;
    }
    // rows of sVt are 8-byte aligned only: two 8-byte stores
    u32x2* pvs = reinterpret_cast<u32x2*>(&sVt[buf][v_d * LDV + c8]);
    pvs[0] = u32x2{rv.x, rv.y};
    pvs[1] = u32x2{rv.z, rv.w};
  };

  f32x16 o;
#pragma unroll
  for (int r = 0; r < 16; ++r) o[r] = 0.f;
  float m_run = -__builtin_huge_valf(), l_run = 0.f;

  const int nkt = (N + KT - 1) / KT;
  // Key tiles whose 64 keys are all masked contribute exactly nothing to a row
  // that has an unmasked key anywhere (their probabilities underflow to zero, or
  // are scaled by exactly zero when the first unmasked key raises the running
  // maximum), so they are left out: same bits, fewer tiles - with padded inputs
  // every row skips the padding's tiles.  A row with no unmasked key at all
  // keeps every tile (its softmax is uniform over the masked keys).  The live
  // tiles of the row as a bit mask, for up to 64 tiles.
  uint64_t live = nkt >= 64 ? ~0ull : (1ull << nkt) - 1;
  bool row_dead = false;
  if (mbase && nkt <= 64) {
    uint32_t* sLive = reinterpret_cast<uint32_t*>(&sK[1][0]);  // not yet in use
    if (tid < 2) sLive[tid] = 0u;
    lds_barrier();
    for (int t0 = 0; t0 < nkt; t0 += 4) {
      const int tile = t0 + wave, key = tile * KT + lane;
      const float mv = *reinterpret_cast<const float*>(mbase + (uint32_t)min(key, N - 1) * 4u);
      const bool on = key < N && mv != 0.f;
      if (__ballot(on) != 0ull && lane == 0) atomicOr(&sLive[tile >> 5], 1u << (tile & 31));
    }
    lds_barrier();
    const uint64_t m = (uint64_t)sLive[0] | ((uint64_t)sLive[1] << 32);
    lds_barrier();  // sLive is read; the buffer may be written
    if (m != 0ull) live = m;
    else row_dead = true;
  }
  const uint32_t live_lo = __builtin_amdgcn_readfirstlane((uint32_t)live);
  const uint32_t live_hi = __builtin_amdgcn_readfirstlane((uint32_t)(live >> 32));
  uint64_t rest = (uint64_t)live_lo | ((uint64_t)live_hi << 32);
  // next live tile, or nkt (a tile past the end: clamped loads, every key at -inf, never used) when none is
  // left; more than 64 tiles (N > 4096) are simply taken in order
  int seq = 0;
  auto pop = [&]() {
    if (nkt > 64) return seq < nkt ? seq++ : nkt;
    if (rest == 0ull) return nkt;
    const int tile = __builtin_ctzll(rest);
    rest &= rest - 1;
    return tile;
  };
  int t_cur = pop(), t_nxt = pop();
  if (row_dead) {
    // Every key of the row is masked: the reference replaces all logits by the
    // same -1e9, the softmax is exactly uniform and every query's output is the
    // mean of V over the N keys (times its gate).  No attention to compute.
    float* sMean = reinterpret_cast<float*>(&sK[0][0]);
    const bf16_t* vrow = a.vt + (bh * D + v_d) * a.ldn;
    float acc = 0.f;
    for (int k0 = c8; k0 < N; k0 += 64) {  // rows of V^T hold ldn >= N keys, ldn a multiple of 8
      float f[8];
      unpack8(*reinterpret_cast<const u32x4*>(vrow + k0), f);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc += k0 + e < N ? f[e] : 0.f;
    }
    acc += __shfl_xor(acc, 1);
    acc += __shfl_xor(acc, 2);
    acc += __shfl_xor(acc, 4);
    if ((tid & 7) == 0) sMean[v_d] = acc;
    lds_barrier();
#pragma unroll
    for (int r = 0; r < 16; ++r) o[r] = sMean[8 * (r >> 2) + 4 * hh + (r & 3)];
    l_run = (float)N;
    t_cur = nkt;  // no tile loop
  } else {
  gload_kv(t_cur * KT);
  gload_bias(rb, t_cur);
  sstore(0);
  gload_kv(t_nxt * KT);
  lds_barrier();
  }

  for (int kt = 0; t_cur < nkt; ++kt) {
    const int buf = kt & 1;
    const int t_nn = pop();
    // The next live tile, fetched during the previous iteration, goes to the
    // other buffer (last read in the previous iteration, which every wave left
    // through the barrier at its end); its registers then take the tile after
    // it.  Past the last tile both are clamped re-reads whose stores nobody reads.
    sstore(buf ^ 1);
    gload_kv(t_nn * KT);
    // Both 32-key halves of the tile go through the matrix unit first (two
    // independent accumulator chains), then one online-softmax update covers
    // all 64 keys, then both halves feed O.  A half that lies wholly beyond N
    // has every key at -inf (mask column) and contributes exactly zero.
    // s[u][4g + e] <-> key 32u + 8g + 4hh + e of this tile, query j.
    f32x16 s[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[u][r] = 0.f;
      if (HAS_BIAS) {
        s[u] = mfma32(idf[0], as_frag(rb[2 * u]), s[u]);
        s[u] = mfma32(idf[1], as_frag(rb[2 * u + 1]), s[u]);
      }
#pragma unroll
      for (int ks = 0; ks < 3; ++ks)
        s[u] = mfma32(lds_frag(sK[buf], LDK, u * 32, ks * 16, lane), qf[ks], s[u]);
    }
    // The next tile's bias is fetched here, behind the score MFMAs, when its
    // registers are free again; like the K / V loads at the top of the loop it
    // is first looked at at the top of the next iteration.
    gload_bias(rb, t_nxt);
    // maximum of the lane's 32 scores as a tree of three-input maxima (16 instructions, depth 4)
    float t3[11];
#pragma unroll
    for (int i = 0; i < 10; ++i) {
      const int e = 3 * i;
      t3[i] = fmaxf(fmaxf(s[e >> 4][e & 15], s[(e + 1) >> 4][(e + 1) & 15]), s[(e + 2) >> 4][(e + 2) & 15]);
    }
    t3[10] = fmaxf(s[1][14], s[1][15]);
    const float t9a = fmaxf(fmaxf(t3[0], t3[1]), t3[2]), t9b = fmaxf(fmaxf(t3[3], t3[4]), t3[5]);
    const float t9c = fmaxf(fmaxf(t3[6], t3[7]), t3[8]), t9d = fmaxf(t3[9], t3[10]);
    float mx = fmaxf(fmaxf(fmaxf(t9a, t9b), t9c), t9d);
    mx = fmaxf(mx, half_swap(xaddr, mx));
    const float m_new = fmaxf(m_run, mx);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    m_run = m_new;
    bf16x8 pf[2][2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        float pv8[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) pv8[e] = __builtin_amdgcn_exp2f(s[u][8 * half + e] - m_new);
        pf[u][half] = as_frag(pack8(pv8));
      }
    // Row sums on the matrix unit: ones * P sums the bf16 probabilities of all
    // 64 keys of the tile, both half-waves' keys included, into every row of
    // the result (32 vector adds and a cross-lane exchange less, 20 registers less).
    f32x16 lsum;
#pragma unroll
    for (int r = 0; r < 16; ++r) lsum[r] = 0.f;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int half = 0; half < 2; ++half) lsum = mfma32(onesf, pf[u][half], lsum);
    l_run = l_run * alpha + lsum[0];
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int r = 0; r < 16; ++r) o[r] *= alpha;
    }
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const bf16_t* vp = &sVt[buf][j * LDV + u * 32 + 16 * half + 4 * hh];
        const u32x2 lo = *reinterpret_cast<const u32x2*>(vp);
        const u32x2 hi = *reinterpret_cast<const u32x2*>(vp + 8);
        u32x4 vv;
        vv.x = lo.x; vv.y = lo.y; vv.z = hi.x; vv.w = hi.y;
        o = mfma32(as_frag(vv), pf[u][half], o);
      }
    lds_barrier();
    t_cur = t_nxt;
    t_nxt = t_nn;
  }

  const float inv = 1.f / l_run;  // l_run already holds the sum over both half-waves' keys
  if (qw >= N) return;
  const bf16_t* gp = a.g + (bh * N + qw) * D + 4 * hh;
  bf16_t* op = a.og + ((int64_t)b * N + qw) * 128 + h * D + 4 * hh;
  u32x2 gw[4];  // all gate loads before the first store (which they could alias as far as the compiler knows)
#pragma unroll
  for (int g = 0; g < 4; ++g) gw[g] = *reinterpret_cast<const u32x2*>(gp + 8 * g);
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    u32x2 w;
    w.x = pack2bf(o[4 * g] * inv * bflo(gw[g].x), o[4 * g + 1] * inv * bfhi(gw[g].x));
    w.y = pack2bf(o[4 * g + 2] * inv * bflo(gw[g].y), o[4 * g + 3] * inv * bfhi(gw[g].y));
    *reinterpret_cast<u32x2*>(op + 8 * g) = w;
  }
}

bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

int launch_triattn_proj(const TriAttnProjArgs& a, hipStream_t stream) {
  if (a.N <= 0 || !a.pair || !a.w_qkvg || !a.q || !a.k || !a.vt || !a.g) return AF3_ERR_BAD_ARG;
  if (a.ldn < a.N || (a.ldn & 7)) return AF3_ERR_BAD_ARG;
  if (a.n_bias != 0 && (a.n_bias != H || !a.w_bias || !a.bias)) return AF3_ERR_BAD_ARG;
  if (!al16(a.pair) || !al16(a.w_qkvg) || !al16(a.w_bias) || !al16(a.q) || !al16(a.k) || !al16(a.vt) ||
      !al16(a.g) || !al16(a.bias))
    return AF3_ERR_BAD_ARG;
  const int64_t tiles = (int64_t)a.N * ((a.N + TM - 1) / TM);
  if (tiles > 0x7fffffff) return AF3_ERR_BAD_ARG;
  if (a.io_f32) hipLaunchKernelGGL(triattn_proj_kernel<float>, dim3((unsigned)tiles), dim3(256), 0, stream, a);
  else hipLaunchKernelGGL(triattn_proj_kernel<bf16_t>, dim3((unsigned)tiles), dim3(256), 0, stream, a);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

int launch_triattn_flash(const TriAttnArgs& a, hipStream_t stream) {
  if (!a.q || !a.k || !a.vt || !a.g || !a.og || a.N <= 0) return AF3_ERR_BAD_ARG;
  if (a.ldn < a.N || (a.ldn & 7)) return AF3_ERR_BAD_ARG;
  if (!al16(a.q) || !al16(a.k) || !al16(a.vt) || !al16(a.g) || !al16(a.og) || !al16(a.bias)) return AF3_ERR_BAD_ARG;
  const int64_t blocks = ((int64_t)H * a.N + 7) / 8 * 8 * ((a.N + QW - 1) / QW);
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  if (a.bias) hipLaunchKernelGGL(triattn_flash_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
  else hipLaunchKernelGGL(triattn_flash_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}
