// Triangle attention, the flash-attention core (4 heads of 32 channels).
//
// Operands (all produced by triattn_proj_kernel, see kernels.h):
//   Q, K    : bf16 [b][h][s][32]  (Q pre-multiplied by log2(e)/sqrt(32))
//   Vt      : bf16 [b][h][32][ldn], V transposed, ldn = N rounded up to 16, columns
//             permuted inside every aligned group of 16 (tri_vt_pos) so that the 8 keys one
//             lane feeds to a P.V MFMA are 16 contiguous bytes
//   bias    : fp16, pair bias * log2(e) in MFMA-fragment order (tri_bias_offset)
//   mask    : fp32 [N][N] 0/1 or null
//
// What sets the pace on this machine (measured): a wave64 exp2 occupies the SIMD's issue port
// for 8 cycles, any other vector instruction for 4-5, a 32x32x16 MFMA for about 16 of the 32
// cycles it takes in the matrix unit - and vector work of OTHER waves does not issue while a
// wave has an MFMA waiting for the unit.  So vector and matrix work overlap only inside one
// wave's own instruction stream.  The other cost is what a workgroup pulls in from L2 per key
// tile: with every load taken out of the key-tile loop (operands reused, results wrong) the
// kernel runs 30 % faster, 17 % of which remain when the same loads all hit the CU's own
// cache, i.e. are the loads into LDS as such, the rest is the L2 traffic (8 KB of K / V^T per
// row and 4 KB of bias per wave and key tile: 28 GB per launch at 1536 tokens).  The kernel
// is built around both:
//   * one wave = 32 queries of R rows b; lane = one query; S^T = K Q^T so that the softmax
//     reductions are per lane.  The pair bias enters on the matrix unit as well, S^T += I *
//     bias^T with an fp16 identity; its fragments do not depend on the row, so the R rows of a
//     wave share one load of them, straight into registers.  (With the fp32 bias as the
//     accumulators' initial value the kernel ran 35 % slower than without any bias: the bytes
//     the bias brings in from L2 are half of all it loads; hence fp16 and two rows per wave.)
//   * the key mask rides in the product as a third k-step (K side 0 / -1e9 / -inf, Q side 1.0),
//     and so does the softmax's running base: the Q side of the next slot holds -base, so the
//     accumulator comes out as s - base and exp2 takes it as it is.  `base` only moves when a
//     tile's scores leave [-64, 16] relative to it (a wave-uniform, rare branch that rescales
//     O and l by an exact-in-fp32 factor and repeats the tile's score product); for ordinary
//     logits it never moves and the softmax is computed without a single subtraction.
//     The third k-step is left out (wave-uniformly) for a tile of 64 unmasked keys while no
//     lane of the row has moved its base: eight MFMAs per key tile and row (the algorithm's
//     own count) plus the four of the bias.
//   * the probabilities of tile v go into O while the exponentials of tile v+1 are computed:
//     each of those four MFMAs is issued in front of eight exponentials of the same wave, its
//     V^T fragment read from LDS one group ahead.  Row sums are taken from the bf16
//     probabilities by v_dot2c_f32_bf16 against a pair of ones (per lane, i.e. per half of the
//     keys; the halves are added once at the end).
//   * K and V^T tiles go from global memory straight into LDS (global_load_lds_dwordx4: no
//     staging registers, no LDS store instructions), double-buffered per row with one barrier
//     per key tile; unpadded rows with XOR-permuted 16-byte chunks keep the fragment reads
//     conflict-free.
// Key tiles whose 64 keys are masked in every row of the wave are left out (their
// probabilities are exactly zero); a row whose keys are ALL masked gets the reference's exact
// answer, the mean of V, directly.
#include <type_traits>

#include "common.h"
#include "kernels.h"

namespace {

constexpr int H = 4, D = 32;
constexpr int KT = 64;    // keys per tile
constexpr int QW = 128;   // queries per workgroup (32 per wave)
constexpr int TILE_BYTES = KT * D * 2;  // a K tile [64 keys][32] or a V^T tile [32][64 keys], bf16
constexpr uint32_t BF16_ONE = 0x3F80u, BF16_NEG_INF = 0xFF80u, BF16_NEG_1E9 = 0xCE6Eu;
// A tile's scores, relative to the base, may rise to 2^T_HI before the base is moved (fp32 and
// bf16 share their exponent range, so nothing is lost up there); the first tile with an unmasked
// key moves it if its maximum lies below 2^T_LO.  Scores of masked keys sit near -1e9.
constexpr float T_HI = 16.f, T_LO = -64.f, LIVE_MIN = -1e8f;

// 64 lanes x 16 bytes from global memory (wave-uniform base + per-lane byte offset + OFF) to
// 1 KB of LDS at the wave-uniform `dst` + OFF (lane l's bytes land at 16 l).  Issued as inline
// assembly on purpose: the compiler tracks loads into LDS that it can see and, unable to tell
// the buffers apart, makes every later fragment read wait for ALL loads in flight (vmcnt(0)),
// the ones issued a moment ago for the next tile included.  Here each buffer is read only
// after a dma_barrier() that follows the load's issue, which is what makes this safe.
template <int OFF>
__device__ __forceinline__ void dma16(const char* gbase, uint32_t voff, const char* dst) {
  const uint32_t lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)dst;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3"
               :: "s"(lds), "v"(voff), "s"(gbase), "n"(OFF) : "memory", "m0");
}
__device__ __forceinline__ bf16x8 lds16(const char* p) { return as_frag(*reinterpret_cast<const u32x4*>(p)); }

// Workgroup barrier that also waits for this wave's loads, those into LDS and the ordinary ones
// (the bias registers).  The wait is a builtin so that the compiler sees it: it then knows the
// registers have landed and puts no wait of its own in front of their use, where it would also
// wait for the loads into LDS issued since.
__device__ __forceinline__ void dma_barrier() {
  __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

__device__ __forceinline__ float max32(const f32x16& a, const f32x16& b) {
  // maximum of the lane's 32 scores as a tree of three-input maxima
  float t3[11];
#pragma unroll
  for (int i = 0; i < 10; ++i) {
    const int e = 3 * i;
    const float x = e < 16 ? a[e & 15] : b[e & 15];
    const float y = e + 1 < 16 ? a[(e + 1) & 15] : b[(e + 1) & 15];
    const float z = e + 2 < 16 ? a[(e + 2) & 15] : b[(e + 2) & 15];
    t3[i] = fmaxf(fmaxf(x, y), z);
  }
  t3[10] = fmaxf(b[14], b[15]);
  const float t9a = fmaxf(fmaxf(t3[0], t3[1]), t3[2]), t9b = fmaxf(fmaxf(t3[3], t3[4]), t3[5]);
  const float t9c = fmaxf(fmaxf(t3[6], t3[7]), t3[8]), t9d = fmaxf(t3[9], t3[10]);
  return fmaxf(fmaxf(fmaxf(t9a, t9b), t9c), t9d);
}

// acc + the two bf16 values packed in `pair` (v_dot2c_f32_bf16 with a pair of ones)
__device__ __forceinline__ float dot2_ones(uint32_t pair, float acc) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf2;
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf2, pair), __builtin_bit_cast(bf2, 0x3F803F80u), acc, false);
}

// o *= f with every register multiplied in place.  Written as plain C++ inside a rarely taken
// branch, the compiler keeps the accumulator in two register tuples and copies all sixteen
// registers on the path that does NOT multiply, every iteration.
__device__ __forceinline__ void scale_in_place(f32x16& o, float f) {
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    float t = o[e];
    asm volatile("v_mul_f32 %0, %1, %0" : "+v"(t) : "v"(f));
    o[e] = t;
  }
}

template <int R, bool HAS_BIAS>
__global__ __launch_bounds__(256, 2) void triattn_flash_kernel(TriAttnArgs a) {
  // [buffer][row] as separate arrays: a load in flight to one of them provably does not alias
  // a fragment read from another
  __shared__ __attribute__((aligned(1024))) char sK00[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sK01[R > 1 ? TILE_BYTES : 16];
  __shared__ __attribute__((aligned(1024))) char sK10[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sK11[R > 1 ? TILE_BYTES : 16];
  __shared__ __attribute__((aligned(1024))) char sV00[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sV01[R > 1 ? TILE_BYTES : 16];
  __shared__ __attribute__((aligned(1024))) char sV10[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sV11[R > 1 ? TILE_BYTES : 16];
  __shared__ uint32_t sLive[R];      // per row: some key is unmasked
  __shared__ uint8_t sFlag[R * 64];  // per row and key tile (the first 64): 1 = some key unmasked, 3 = all 64 of them
  __shared__ float sMean[D];
  __shared__ uint32_t sRedo;  // a wave's unmasked-tile shortcut went wrong: the workgroup repeats its rows without it
  extern __shared__ __attribute__((aligned(16))) uint16_t sCode[];  // [R][nkt * 64] mask code per key
#define KBUF(ph, r) ((ph) == 0 ? ((r) == 0 ? sK00 : sK01) : ((r) == 0 ? sK10 : sK11))
#define VBUF(ph, r) ((ph) == 0 ? ((r) == 0 ? sV00 : sV01) : ((r) == 0 ? sV10 : sV11))

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hh = lane >> 5, j = lane & 31;
  const int xaddr = half_swap_addr();
  const int N = a.N;
  const int ldn = (int)a.ldn;
  const int QT = (N + QW - 1) / QW;
  const int NG = (N + R - 1) / R;  // groups of R rows
  // Workgroup ids are dealt round-robin to the 8 XCDs.  The query tiles of one (row group,
  // head) share its K / V and run back to back on one XCD; the (row group, head) pairs are
  // dealt to the XCDs in turn, so every XCD works on one head at a time (pair % 4 follows
  // from xcd % 4) and finds that head's bias in its L2.
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int qt = slot % QT;
  const int pair_idx = (slot / QT) * 8 + xcd;
  if (pair_idx >= H * NG) return;
  const int rg = pair_idx / H;
  const int h = pair_idx % H;
  const int q0 = qt * QW;
  const int qw = q0 + wave * 32 + j;
  const int qi = min(qw, N - 1);
  const int nkt = (N + KT - 1) / KT;
  const int nk64 = nkt * KT;

  int brow[R];
  bool bvalid[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    bvalid[r] = rg * R + r < N;
    brow[r] = min(rg * R + r, N - 1);
  }

  // ---- mask pass: per-key codes for the mask k-step, live key tiles, dead rows ----
  if (tid < R) sLive[tid] = 0u;
  if (tid < R * 16) reinterpret_cast<uint32_t*>(sFlag)[tid] = 0u;
  if (tid == 0) sRedo = 0u;
  lds_barrier();
  // A wave takes every fourth key tile; the mask values of eight of its tiles and all rows are
  // requested together (one trip per 32 key tiles, not one per tile and row).  The mask is small
  // and comes out of L2; Q comes from memory and is requested right behind the first batch of
  // mask values: loads return in order, so the mask pass does not wait for it, and it travels
  // while the mask pass, the barriers and the first tiles' loads are under way.
  bf16x8 qf[R][2];
  // What a wave finds out about a tile is one byte in LDS, written by all its lanes alike; the
  // workgroup's bit masks of live and of wholly unmasked tiles are ballots over those bytes.
  bool my_any[R];
#pragma unroll
  for (int r = 0; r < R; ++r) my_any[r] = false;
  for (int t0 = 0; t0 < nkt; t0 += 32) {
    float mv[R][8];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int u = 0; u < 8; ++u)
        mv[r][u] = a.mask ? a.mask[(int64_t)brow[r] * N + min((t0 + 4 * u + wave) * KT + lane, N - 1)] : 1.f;
    if (t0 == 0) {
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int64_t row = ((int64_t)brow[r] * H + h) * N + qi;
        const bf16_t* qp = a.q + row * D + 8 * hh;
        qf[r][0] = as_frag(*reinterpret_cast<const u32x4*>(qp));
        qf[r][1] = as_frag(*reinterpret_cast<const u32x4*>(qp + 16));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int tile = t0 + 4 * u + wave;
        if (tile < nkt) {
          const int key = tile * KT + lane;
          const bool on = key < N && mv[r][u] != 0.f;
          sCode[r * nk64 + key] = (uint16_t)(key >= N ? BF16_NEG_INF : (mv[r][u] == 0.f ? BF16_NEG_1E9 : 0u));
          const uint64_t on_lanes = __ballot(on);
          my_any[r] = my_any[r] || on_lanes != 0ull;
          if (tile < 64) sFlag[r * 64 + tile] = (uint8_t)((on_lanes != 0ull ? 1 : 0) | (on_lanes == ~0ull ? 2 : 0));
        }
      }
  }
#pragma unroll
  for (int r = 0; r < R; ++r)
    if (my_any[r]) sLive[r] = 1u;
  lds_barrier();
  bool dead[R];
  uint64_t live = 0ull;
  uint64_t plain[R];  // tiles of 64 unmasked keys below N (none beyond the 64th tile): they need no mask k-step
  bool all_dead = true;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    dead[r] = __builtin_amdgcn_readfirstlane(sLive[r]) == 0u;
    const uint32_t flag = lane < nkt ? sFlag[r * 64 + lane] : 0u;
    all_dead = all_dead && dead[r];
    live |= __ballot((flag & 1u) != 0u);
    plain[r] = __ballot((flag & 2u) != 0u);
  }
  // next live tile, or nkt when none is left; more than 64 tiles are simply taken in order
  uint64_t rest = live;
  int seq = 0;
  auto pop = [&]() {
    if (nkt > 64) return seq < nkt ? seq++ : nkt;
    if (rest == 0ull) return nkt;
    const int tile = __builtin_ctzll(rest);
    rest &= rest - 1;
    return tile;
  };

  f32x16 o[R];
  float lrun[R], base[R], mrel[R];  // lrun: sum of the probabilities of THIS lane's keys (half of each tile)
#pragma unroll
  for (int r = 0; r < R; ++r) {
#pragma unroll
    for (int e = 0; e < 16; ++e) o[r][e] = 0.f;
    lrun[r] = 0.f;
    base[r] = 0.f;
    mrel[r] = -__builtin_huge_valf();
  }

  if (!all_dead) {
    // ---- per-lane constants ----
    u32x4 qm[R];  // Q side of the mask k-step: slot 0 = 1.0 (times the key's code), slot 1 = -base
    const char* kglob[R];
    const char* vglob[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t bh = (int64_t)brow[r] * H + h;
      qm[r] = u32x4{hh == 0 ? (BF16_ONE | 0x80000000u) : 0u, 0u, 0u, 0u};  // -0.0 in slot 1
      kglob[r] = reinterpret_cast<const char*>(a.k + bh * N * D);
      vglob[r] = reinterpret_cast<const char*>(a.vt + bh * D * a.ldn);
    }
    // fragment reads: K row (32 u + j), chunk (2 ks + hh) ^ ((j >> 2) & 3); V^T row j, chunk (2 s + hh) ^ ((j >> 1) & 7)
    const int ksw = (j >> 2) & 3;
    const int ka0 = j * 64 + ((hh ^ ksw) << 4), ka1 = j * 64 + (((2 + hh) ^ ksw) << 4);
    const int vsw = (j >> 1) & 7;
    int va[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) va[s] = j * 128 + (((2 * s + hh) ^ vsw) << 4);
    // loads into LDS: K keys 16 w + lane / 4, position lane % 4; V^T rows 8 w + lane / 8, position lane % 8
    const int dk_key = 16 * wave + (lane >> 2);
    const uint32_t dk_chunk = (uint32_t)(((lane & 3) ^ ((dk_key >> 2) & 3)) << 4);
    const int dv_row = 8 * wave + (lane >> 3);
    const int dv_col = ((lane & 7) ^ ((dv_row >> 1) & 7)) * 8;
    auto dma_k = [&](int tile, int r, char* buf) {  // a tile past the end re-reads the last one (never used)
      const int key = min(min(tile, nkt - 1) * KT + dk_key, N - 1);
      dma16<0>(kglob[r], (uint32_t)key * (D * 2u) + dk_chunk, buf + wave * 1024);
    };
    auto dma_v = [&](int tile, int r, char* buf) {
      const int col = min(tile, nkt - 1) * KT + dv_col;  // columns past ldn: any finite data will do (P is zero there)
      dma16<0>(vglob[r], (uint32_t)(dv_row * ldn + (col < ldn ? col : 0)) * 2u, buf + wave * 1024);
    };
    // bias tiles of this wave's 32-query block: 4 KB per key tile
    const int wave_blk = q0 + wave * 32 < N ? (q0 >> 5) + wave : 0;
    const char* bbase =
        HAS_BIAS ? reinterpret_cast<const char*>(a.bias + tri_bias_offset(N, h, wave_blk * 32, 0)) : nullptr;
    // The bias tile of key tile t + 1 (four 1 KB fp16 fragments; fragment i = 2 u + st: keys
    // 32 u + 16 st + 8 hh .. + 8 of this lane's query, bytes 32 j + 16 hh of run i) is only ever
    // read by this wave, so it goes from memory straight into registers, requested when tile t
    // begins.  The wait that the barrier in the middle of tile t needs anyway covers it.  While
    // the last row of tile t computes its exponentials the fragments are turned into fp32 on
    // the matrix unit, bt = I * bias^T with an fp16 identity: the initial value of the score
    // accumulators of every row of tile t + 1 (four MFMAs per key tile, each issued between
    // two groups of exponentials).  (Staged through LDS like K and V^T, by loads into LDS two
    // tiles ahead, the same kernel ran 3.5 % slower: a load into LDS costs the wave more than
    // a load into registers, and the fragments cost an LDS read each on top.)
    f32x16 bt[2];
    u32x4 bnext[4];
    auto load_bias = [&](int tile) {
      if (!HAS_BIAS) return;
      const char* p = bbase + (size_t)min(tile, nkt - 1) * 4096u + (j * 32 + hh * 16);
#pragma unroll
      for (int i = 0; i < 4; ++i) bnext[i] = *reinterpret_cast<const u32x4*>(p + 1024 * i);
    };
    // Identity fragments (fp16): A-fragment of k-step st: lane (row i = j, half hh) holds
    // I[i][16 st + 8 hh + e], e = 0..7: a single 1.0 where 16 st + 8 hh + e == i.
    f16x8 idf[2];
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const int e1 = j - 16 * st - 8 * hh;
      uint32_t w[4] = {0u, 0u, 0u, 0u};
      if (e1 >= 0 && e1 < 8) w[e1 >> 1] = (e1 & 1) ? (0x3C00u << 16) : 0x3C00u;
      idf[st] = as_frag_f16(u32x4{w[0], w[1], w[2], w[3]});
    }
    f32x16 zero16;
#pragma unroll
    for (int e = 0; e < 16; ++e) zero16[e] = 0.f;
    // scores of one row's virtual tile: the two halves of the head dimension on top of the bias
    auto scores = [&](const bf16x8& k00, const bf16x8& k01, const bf16x8& k10, const bf16x8& k11, const bf16x8* q,
                      f32x16& s0, f32x16& s1) {
      s0 = mfma32(k00, q[0], bt[0]);
      s1 = mfma32(k10, q[0], bt[1]);
      s0 = mfma32(k01, q[1], s0);
      s1 = mfma32(k11, q[1], s1);
    };
#pragma unroll
    for (int e = 0; e < 16; ++e) bt[0][e] = bt[1][e] = 0.f;
    bool based[R];  // some lane of the wave has moved this row's base off zero
    float pend_alpha = 1.f;  // R == 1: a rescaling of O and l that waits for the tile in flight
    bool pend = false;
    // Tiles of 64 unmasked keys take their exponentials without looking at the tile's maximum
    // first ("fast").  Every lane of such a tile has 32 live keys, so the sums of what it got say
    // afterwards where the scores lay: a tile sum that is not below 2^60 (an overflow included)
    // means scores far above the base, a row total below 2^-30 scores far below it.  Per tile
    // only the largest tile sum is kept (one instruction); both conditions are looked at once,
    // when the row is through.  Either is rare and makes the whole workgroup repeat its rows
    // with every tile on the careful route.
    bool allow_fast = true;
    uint64_t bad = 0ull;
    float lmax[R];      // largest sum of one fast tile
    bool used_fast[R];  // this wave took some tile of the row the fast way
    bf16x8 kpre[4];  // R == 2: row 0's K fragments of the next key tile
    u32x4 pp[4];  // probabilities of the previous virtual tile (bf16 B fragments), zero before the first

    // One virtual tile = (key tile, row RR): scores, softmax, and meanwhile the previous
    // virtual tile's probabilities go into its row sums and its O.
    auto iter = [&](auto PHc, auto RRc, int tile) {
      constexpr int PH = decltype(PHc)::value, RR = decltype(RRc)::value;
      constexpr int PR = (RR + R - 1) % R, VPH = RR == 0 ? PH ^ 1 : PH;
      const char* kb = KBUF(PH, RR);
      const char* vb = VBUF(VPH, PR);
      if (R == 1 && pend) {
        scale_in_place(o[0], pend_alpha);
        pend = false;
      }
      // The third k-step carries the key mask and the base.  A tile of 64 unmasked keys whose row
      // still has base 0 in every lane needs neither (wave-uniform).
      const bool fast = allow_fast && tile < 64 && ((plain[RR] >> tile) & 1ull) != 0ull;
      const bool step3 = based[RR] || !fast;
      // Two rows per wave: row 0's K tile has been in LDS since the barrier before the previous
      // virtual tile, whose last group of exponentials fetched these fragments (kpre).
      const bool pre = R == 2 && RR == 0;
      const bf16x8 k00 = pre ? kpre[0] : lds16(kb + ka0), k01 = pre ? kpre[1] : lds16(kb + ka1);
      const bf16x8 k10 = pre ? kpre[2] : lds16(kb + 2048 + ka0), k11 = pre ? kpre[3] : lds16(kb + 2048 + ka1);
      bf16x8 af0, af1;
      f32x16 s0, s1;
      scores(k00, k01, k10, k11, qf[RR], s0, s1);
      if (step3) {
        const uint16_t* mc = sCode + RR * nk64 + tile * KT;
        const uint32_t c0 = mc[j], c1 = mc[32 + j];
        af0 = as_frag(u32x4{hh == 0 ? (c0 | (BF16_ONE << 16)) : 0u, 0u, 0u, 0u});
        af1 = as_frag(u32x4{hh == 0 ? (c1 | (BF16_ONE << 16)) : 0u, 0u, 0u, 0u});
        s0 = mfma32(af0, as_frag(qm[RR]), s0);
        s1 = mfma32(af1, as_frag(qm[RR]), s1);
      }

      if (!fast) {
      float mx = max32(s0, s1);
      mx = fmaxf(mx, half_swap(xaddr, mx));
      const float mnew = fmaxf(mrel[RR], mx);
      // (lanes of queries past the end have no say: in a partly filled block they see bias values nobody wrote)
      const bool want = qw < N && (mx > T_HI || (mnew < T_LO && mnew > LIVE_MIN));
      if (__any(want)) {
        // Move the base of every query of the wave to its running maximum (rounded to bf16, the
        // form the matrix unit takes it in), rescale what the row has accumulated, and repeat the
        // score product.  Lanes that have seen no unmasked key yet keep their base: their O and l
        // are still exactly zero.
        const bool has_live = mnew > LIVE_MIN;
        const float nb = has_live ? bf2f(f2bf(base[RR] + mnew)) : base[RR];
        const float delta = nb - base[RR];
        const float alpha = mrel[RR] > LIVE_MIN ? __builtin_amdgcn_exp2f(-delta) : 1.f;
        base[RR] = nb;
        mrel[RR] = mnew - delta;
        qm[RR].x = hh == 0 ? (BF16_ONE | ((uint32_t)f2bf(-nb) << 16)) : 0u;
        based[RR] = true;
        if (!step3) {
          const uint16_t* mc = sCode + RR * nk64 + tile * KT;
          const uint32_t c0 = mc[j], c1 = mc[32 + j];
          af0 = as_frag(u32x4{hh == 0 ? (c0 | (BF16_ONE << 16)) : 0u, 0u, 0u, 0u});
          af1 = as_frag(u32x4{hh == 0 ? (c1 | (BF16_ONE << 16)) : 0u, 0u, 0u, 0u});
        }
        lrun[RR] *= alpha;  // the row sums are up to date (taken when the probabilities are made)
        if (R == 1) {
          // the previous virtual tile belongs to the same row and its probabilities, relative to the
          // old base, are not in O yet: O gets the factor once they are (top of the next iteration)
          pend_alpha = alpha;
          pend = true;
        } else {
          scale_in_place(o[RR], alpha);
        }
        scores(k00, k01, k10, k11, qf[RR], s0, s1);
        s0 = mfma32(af0, as_frag(qm[RR]), s0);
        s1 = mfma32(af1, as_frag(qm[RR]), s1);
      } else {
        mrel[RR] = mnew;
      }
      }
      float linc = 0.f;
      // From here to the end: one basic block in a fixed order.  Each of the four P.V MFMAs of the
      // previous virtual tile is issued in front of eight exponentials of this one (the matrix
      // unit works while the wave goes on issuing vector instructions; another wave's would not
      // get in), with its V^T fragment read from LDS one group ahead.
      bf16x8 vf = lds16(vb + va[0]);
      u32x4 bfr[4];  // the next key tile's bias fragments (the last row of this one fetches them)
      if (HAS_BIAS && RR == R - 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) bfr[i] = bnext[i];  // (the registers are free for the next request)
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const bf16x8 vcur = vf;
        if (s < 3) {
          vf = lds16(vb + va[s + 1]);
          __builtin_amdgcn_sched_barrier(0);
        } else if (R == 2 && RR == 1) {
          const char* kn = KBUF(PH ^ 1, 0);
          kpre[0] = lds16(kn + ka0);
          kpre[1] = lds16(kn + ka1);
          kpre[2] = lds16(kn + 2048 + ka0);
          kpre[3] = lds16(kn + 2048 + ka1);
          __builtin_amdgcn_sched_barrier(0);
        }
        o[PR] = mfma32(vcur, as_frag(pp[s]), o[PR]);
        float p8[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) p8[e] = __builtin_amdgcn_exp2f(s < 2 ? s0[8 * (s & 1) + e] : s1[8 * (s & 1) + e]);
        if (HAS_BIAS && RR == R - 1) {
          // fragments 2 u + st: bt[u] = I(st = 0) * f(2 u) + I(st = 1) * f(2 u + 1); group s does (u, st) = (s / 2, s % 2)
          asm volatile("" : "+v"(p8[0]), "+v"(p8[1]), "+v"(p8[2]), "+v"(p8[3]));
          bt[s >> 1] = mfma32_f16(idf[s & 1], as_frag_f16(bfr[s]), (s & 1) ? bt[s >> 1] : zero16);
        }
#pragma unroll
        for (int e = 4; e < 8; ++e) p8[e] = __builtin_amdgcn_exp2f(s < 2 ? s0[8 * (s & 1) + e] : s1[8 * (s & 1) + e]);
        // this tile's probabilities take the place of the previous tile's, whose last reader (the
        // MFMA above) has been issued
        pp[s] = pack8(p8);
        // pins the exponentials to this group (without it they sink to where their values are used,
        // the next iteration's MFMAs)
        asm volatile("" : "+v"(pp[s].x), "+v"(pp[s].y), "+v"(pp[s].z), "+v"(pp[s].w));
        linc = dot2_ones(pp[s].w, dot2_ones(pp[s].z, dot2_ones(pp[s].y, dot2_ones(pp[s].x, linc))));
        __builtin_amdgcn_sched_barrier(0);
      }
      lrun[RR] += linc;
      if (fast) {
        lmax[RR] = fmaxf(lmax[RR], linc);
        // If the row passes its check at the end, its total is at least 2^-30 over at most 4096
        // keys: a lower bound of the running maximum, all the careful route's lower guard needs
        // (if it does not, the rows are repeated and what a careful tile decided meanwhile is void).
        mrel[RR] = fmaxf(mrel[RR], -42.f);
        used_fast[RR] = true;
      }
    };
    // the tail of the pipeline: the last virtual tile's probabilities
    auto drain = [&](const char* vb) {
      constexpr int PR = R - 1;
      if (R == 1 && pend) scale_in_place(o[0], pend_alpha);  // what was accumulated before the last tile moved the base
#pragma unroll
      for (int s = 0; s < 4; ++s) o[PR] = mfma32(lds16(vb + va[s]), as_frag(pp[s]), o[PR]);
    };

#pragma nounroll
    for (int pass = 0; pass < 2; ++pass) {
    allow_fast = pass == 0;
    bad = 0ull;
    rest = live;
    seq = 0;
    pend = false;
#pragma unroll
    for (int s = 0; s < 4; ++s) pp[s] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
      for (int e = 0; e < 16; ++e) o[r][e] = 0.f;
      lrun[r] = 0.f;
      base[r] = 0.f;
      mrel[r] = -__builtin_huge_valf();
      qm[r].x = hh == 0 ? (BF16_ONE | 0x80000000u) : 0u;
      based[r] = false;
      lmax[r] = 0.f;
      used_fast[r] = false;
    }
    int t_cur = pop(), t_n1 = pop(), t_n2 = pop();
    // the buffer the first virtual tile reads its "previous" V^T from must hold finite data
    *reinterpret_cast<u32x4*>(VBUF(1, R - 1) + tid * 16) = u32x4{0u, 0u, 0u, 0u};
    // the first tiles' loads into LDS and the first bias tile's ordinary loads travel together
    dma_k(t_cur, 0, KBUF(0, 0));
    if (R == 2) {
      dma_k(t_cur, 1, KBUF(0, 1));
      dma_k(t_n1, 0, KBUF(1, 0));
      dma_v(t_cur, 0, VBUF(0, 0));
      dma_v(t_cur, 1, VBUF(0, 1));
    }
    if (HAS_BIAS) {
      const char* p = bbase + (size_t)t_cur * 4096u + (j * 32 + hh * 16);
      u32x4 f[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) f[i] = *reinterpret_cast<const u32x4*>(p + 1024 * i);
      bt[0] = mfma32_f16(idf[1], as_frag_f16(f[1]), mfma32_f16(idf[0], as_frag_f16(f[0]), zero16));
      bt[1] = mfma32_f16(idf[1], as_frag_f16(f[3]), mfma32_f16(idf[0], as_frag_f16(f[2]), zero16));
    }
    if (R == 2) {
      dma_barrier();
      kpre[0] = lds16(KBUF(0, 0) + ka0);
      kpre[1] = lds16(KBUF(0, 0) + ka1);
      kpre[2] = lds16(KBUF(0, 0) + 2048 + ka0);
      kpre[3] = lds16(KBUF(0, 0) + 2048 + ka1);
    }
    // Every ordinary load issued so far (Q, the first bias tile) is waited for HERE, with a wait
    // the compiler can see: otherwise it keeps a vmcnt(0) for them at the top of the loop, where
    // it would also wait, every iteration, for the loads into LDS issued just before.
    __builtin_amdgcn_s_waitcnt(0x0F70);
    // One key tile per step.  R = 2: row 0's virtual tile, barrier, loads for what is read
    // after the NEXT barrier (K of row 1 of the next tile, K of row 0 of the tile after it,
    // V^T of the next tile), row 1's virtual tile.  R = 1: barrier, loads (next K, this V^T),
    // the virtual tile.
    auto step = [&](auto PHc) {
      constexpr int PH = decltype(PHc)::value;
      using P0 = std::integral_constant<int, PH>;
      if (R == 2) {
        load_bias(t_n1);
        iter(P0{}, std::integral_constant<int, 0>{}, t_cur);
        dma_barrier();
        dma_k(t_n1, 1, KBUF(PH ^ 1, 1));
        dma_k(t_n2, 0, KBUF(PH, 0));
        dma_v(t_n1, 0, VBUF(PH ^ 1, 0));
        dma_v(t_n1, 1, VBUF(PH ^ 1, 1));
        iter(P0{}, std::integral_constant<int, R - 1>{}, t_cur);
      } else {
        dma_barrier();
        load_bias(t_n1);  // R == 1: requested behind the barrier, used at the end of this virtual tile
        dma_k(t_n1, 0, KBUF(PH ^ 1, 0));
        dma_v(t_cur, 0, VBUF(PH, 0));
        iter(P0{}, std::integral_constant<int, 0>{}, t_cur);
      }
      t_cur = t_n1;
      t_n1 = t_n2;
      t_n2 = pop();
    };
    int last_ph = 0;
    while (true) {
      step(std::integral_constant<int, 0>{});
      last_ph = 0;
      if (t_cur >= nkt) break;
      step(std::integral_constant<int, 1>{});
      last_ph = 1;
      if (t_cur >= nkt) break;
    }
    dma_barrier();  // every load into LDS has landed (none is in flight when the workgroup ends)
    drain(last_ph == 0 ? VBUF(0, R - 1) : VBUF(1, R - 1));
    if (pass == 1) break;
    // (lanes of queries past the end work on clamped operands and, in a partly filled bias block, on
    // bias values nobody wrote: they have no say)
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (!used_fast[r] || dead[r]) continue;
      const float lt = lrun[r] + half_swap(xaddr, lrun[r]);
      bad |= __ballot(qw < N && (!(lmax[r] < 0x1p60f) || lt < 0x1p-30f));
    }
    if (bad != 0ull && lane == 0) sRedo = 1u;
    lds_barrier();  // also: every wave is done with the K / V^T tiles before a second pass loads over them
    if (__builtin_amdgcn_readfirstlane(sRedo) == 0u) break;
    }
  }

  // a query's keys are split over the two half-waves
#pragma unroll
  for (int r = 0; r < R; ++r) lrun[r] += half_swap(xaddr, lrun[r]);

  // ---- rows whose keys are all masked: the reference replaces every logit by the same -1e9,
  // the softmax is exactly uniform and each query's output is the mean of V over the N keys ----
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (!dead[r]) continue;
    lds_barrier();
    const int v_d = tid >> 3, c8 = (tid & 7) * 8;
    const bf16_t* vrow = a.vt + (((int64_t)brow[r] * H + h) * D + v_d) * a.ldn;
    float acc = 0.f;
    // columns N..ldn-1 are zero; eight loads in flight at a time (one at a time, each waits out a
    // trip to memory, and a row of padding costs as much as a row of attention)
    for (int kb = c8; kb < ldn; kb += 512) {
      u32x4 raw[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int k0 = kb + 64 * i;
        raw[i] = *reinterpret_cast<const u32x4*>(vrow + (k0 < ldn ? k0 : c8));
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float f[8];
        unpack8(raw[i], f);
        if (kb + 64 * i < ldn) {
#pragma unroll
          for (int e = 0; e < 8; ++e) acc += f[e];
        }
      }
    }
    acc += __shfl_xor(acc, 1);
    acc += __shfl_xor(acc, 2);
    acc += __shfl_xor(acc, 4);
    if ((tid & 7) == 0) sMean[v_d] = acc;
    lds_barrier();
#pragma unroll
    for (int e = 0; e < 16; ++e) o[r][e] = sMean[8 * (e >> 2) + 4 * hh + (e & 3)];
    lrun[r] = (float)N;
  }

  if (qw >= N) return;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (!bvalid[r]) continue;
    const float inv = 1.f / lrun[r];  // the sum over both half-waves' keys
    bf16_t* op = a.og + ((int64_t)brow[r] * N + qw) * 128 + h * D + 4 * hh;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 w;
      w.x = pack2bf(o[r][4 * g] * inv, o[r][4 * g + 1] * inv);
      w.y = pack2bf(o[r][4 * g + 2] * inv, o[r][4 * g + 3] * inv);
      *reinterpret_cast<u32x2*>(op + 8 * g) = w;
    }
  }
#undef KBUF
#undef VBUF
}

bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

int launch_triattn_flash(const TriAttnArgs& a, hipStream_t stream) {
  if (!a.q || !a.k || !a.vt || !a.og || a.N <= 0 || a.N > 8192) return AF3_ERR_BAD_ARG;
  if (a.ldn < a.N || (a.ldn & 15)) return AF3_ERR_BAD_ARG;
  if (!al16(a.q) || !al16(a.k) || !al16(a.vt) || !al16(a.og) || !al16(a.bias)) return AF3_ERR_BAD_ARG;
  const int QT = (a.N + QW - 1) / QW;
  const int nkt = (a.N + KT - 1) / KT;
  // Two rows per wave once that still leaves every CU several workgroups, one row below that
  // (and when the per-key mask codes of two rows would not fit the LDS share of a workgroup).
  int R = (int64_t)((a.N + 1) / 2) * H * QT >= 2048 ? 2 : 1;
  // static LDS: K / V buffers, small arrays; dynamic: the mask codes.  Two workgroups must fit a
  // CU's 160 KB.
  const size_t stat2 = 8 * TILE_BYTES + 512;
  if (R == 2 && stat2 + 2 * (size_t)nkt * KT * sizeof(uint16_t) > 80 * 1024) R = 1;
  const int NG = (a.N + R - 1) / R;
  const int64_t blocks = ((int64_t)H * NG + 7) / 8 * 8 * QT;
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  const size_t dyn = (size_t)R * nkt * KT * sizeof(uint16_t);
  const dim3 grid((unsigned)blocks), block(256);
  const size_t stat = (R == 2 ? 8 : 4) * TILE_BYTES + 512;
  auto launch = [&](void (*kernel)(TriAttnArgs)) {
    // more than 64 KB of LDS per workgroup in all (static + dynamic) has to be asked for
    // (a per-function, per-device setting of the runtime: no allocation, no synchronisation)
    if (stat + dyn > 65536) {
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)dyn);
      (void)hipGetLastError();
    }
    hipLaunchKernelGGL(kernel, grid, block, dyn, stream, a);
  };
  if (R == 2) {
    if (a.bias) launch(triattn_flash_kernel<2, true>);
    else launch(triattn_flash_kernel<2, false>);
  } else {
    if (a.bias) launch(triattn_flash_kernel<1, true>);
    else launch(triattn_flash_kernel<1, false>);
  }
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}
