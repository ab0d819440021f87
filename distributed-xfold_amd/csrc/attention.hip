// Flash-style pair-biased attention on bf16 MFMA; the [B, H, Sq, Sk] logits
// never reach HBM.
//
// One wave owns 32 queries of one (batch, head).  Logits are computed
// TRANSPOSED, S^T = K Q^T, so that in the MFMA accumulator layout a lane owns
// one query (column) and 16 of the 32 keys of a tile (rows): the online-softmax
// row maximum / row sum are then in-register reductions plus one exchange
// between the two lane halves.  The same registers, rounded to bf16, are
// directly the B fragments of O^T += V^T P^T (the MFMA k index is a summation
// index, so the key order inside a fragment is free as long as the V^T
// fragment uses the same order).  K and V tiles of 64 keys are staged in LDS row
// by row as they lie in memory, double-buffered and shared by the workgroup's
// waves; the V^T fragments come out of the transposing LDS read of this target
// (ds_read_b64_tr_b16), so nothing is transposed on the way in.
//
// Logit = q.k (q pre-scaled) + pair_bias[h][q][k]; then
//   key_mask:  keys with mask 0 are REPLACED by -1e9 (so a fully masked row is
//              uniform over all Sk keys, like the reference's masked_fill);
//   qpad/kpad: +1e9 where both the query and the key are padding (the atom
//              cross-attention convention).
// Keys beyond Sk (tile padding) get -inf and never contribute.
#include "common.h"
#include "kernels.h"

namespace {

constexpr int KT = 64;        // keys per LDS tile
constexpr float NEG_INF = -__builtin_huge_valf();
typedef short v4s __attribute__((ext_vector_type(4)));
typedef short v8s __attribute__((ext_vector_type(8)));
// ds_read_b64_tr_b16: four 16-bit elements per lane, transposed within each group of 16 lanes
__device__ __forceinline__ v4s lds_read_tr16(const bf16_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)p);
}
constexpr float LOG2E = 1.4426950408889634f;
// per-key code staged in LDS next to the K tile
constexpr int KEY_MASKED = 1, KEY_PAD = 2, KEY_BEYOND = 4;

// FAST: keys are rows of K / V as they stand (no row table) and the pair bias is present and 16-byte
// addressable.  Then every address of the key-tile loop is a wave-uniform base that advances by a
// constant per tile plus a per-lane offset that never changes, and the bias quads are loaded straight
// into the registers in which the matrix unit accumulates K Q^T on top of them: no address arithmetic
// and no bias additions in the loop.  The last tile of a key count that is not a multiple of 64 takes
// the clamped addresses of the general form.
template <int KSTEPS, int DVT, int NW, bool FAST>
// at least two waves per SIMD: the register allocator then keeps everything in
// the 256 architectural VGPRs instead of parking loop state in accumulation
// registers, which would leave a single wave per SIMD (the one-wave workgroup of
// head dimension 48 stages twelve chunks per thread and is given the whole register file)
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(KSTEPS == 3 && NW == 1 ? 1 : 2)))
void flash_kernel(FlashArgs a) {
  constexpr int KD = KSTEPS * 16;  // padded q/k head dim
  constexpr int LDK = KD + 8;      // sK row stride (bf16)
  constexpr int NT = NW * 64;
  __shared__ __attribute__((aligned(16))) bf16_t sK[2][KT * LDK];
  // sV row stride (bf16): V rows as they are, padded to the 32 DVT columns the products read.  A transposing
  // read touches 8 rows x 64 bytes; with a row stride of 16 or 48 dwords modulo the 64 banks (32 or 96
  // elements) these tile the banks exactly twice, the minimum for its 512 bytes.
  constexpr int LDV = DVT == 1 ? 32 : 96;
  static_assert(LDV >= DVT * 32, "a row holds every column the products read");
  __shared__ __attribute__((aligned(16))) bf16_t sV[2][KT * LDV];
  __shared__ __attribute__((aligned(16))) int sCode[2][KT];
  __shared__ int sAnyCode[2];  // whether any key of the staged tile carries a code

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hh = lane >> 5, j = lane & 31;
  const int xaddr = half_swap_addr();
  // Batch entries that share a slab of a non-batched pair bias must meet in one L2 for that slab to be
  // fetched from memory once: workgroup ids are dealt round-robin to the 8 XCDs, each with an L2 of its
  // own, so id -> (xcd, slot) -> logical id gives every XCD a contiguous range of logical ids, and
  // logical = (q_tile * H + head) * B + batch has the sharing entries as its fastest index.
  int b, h, q0;
  if (a.bias_mod > 0) {
    // (windows of a few keys: the workgroups are short and the bias slabs small; plain order)
    if ((int)blockIdx.x >= a.n_blocks) return;
    b = blockIdx.x % a.B;
    h = (blockIdx.x / a.B) % a.H;
    q0 = (blockIdx.x / (a.B * a.H)) * (NW * 32) + wave * 32;
  } else {
    const int per_xcd = (gridDim.x + 7) >> 3;
    const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (logical >= a.n_blocks) return;  // workgroup-uniform, before any barrier
    b = logical % a.B;
    h = (logical / a.B) % a.H;
    q0 = (logical / (a.B * a.H)) * (NW * 32) + wave * 32;
  }
  const int d = a.d;
  const int qi = min(q0 + j, a.Sq - 1);  // clamped for loads; stores are guarded
  const bool q_ok = q0 + j < a.Sq;

  // Q^T fragments: lane (query j, half hh) holds head-dim 16*ks + 8*hh .. +7
  bf16x8 qf[KSTEPS];
  {
    const bf16_t* qp = a.q + (int64_t)b * a.q_sb + (int64_t)qi * a.q_ss + h * d;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const int c = 16 * ks + 8 * hh;
      const u32x4 z = {0, 0, 0, 0};
      const u32x4 v = *reinterpret_cast<const u32x4*>(qp + (c < d ? c : 0));
      qf[ks] = as_frag(c < d ? v : z);
    }
  }
  const bf16x8 onesf = as_frag(u32x4{0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u});

  // With key_rows, K / V are tables of rows shared by bias_mod consecutive batch
  // entries (one table per sample) and the key rows of this batch entry are
  // looked up in key_rows; a negative entry is a key whose K and V rows are zero.
  const int64_t kv_b = a.key_rows ? b / a.bias_mod : b;
  const bf16_t* kg = a.k + kv_b * a.k_sb + h * d;
  const bf16_t* vg = a.v + kv_b * a.v_sb + h * d;
  const int dch = d / 8;  // 16-byte chunks per real key row

  // Tile loaders (global -> registers -> LDS).  Every load is unconditional,
  // from a clamped address, and nothing is decided from a loaded value before
  // the LDS store one tile later: a load under a lane mask, or a value
  // inspected right after its load, costs a full memory round trip per tile.
  //   chunk id = key * (KD/8) + c, c fastest (one key row is contiguous), for K and for V alike: both go to
  //   LDS row by row as they lie in memory
  // The K chunks of a tile and then its V chunks form one list of 2 KCH entries that the threads share out
  // evenly: thread t moves entries t, t + NT, ..  (head dimension 48 with 256 threads: three each, the
  // middle one a K chunk for waves 0 and 1 and a V chunk for waves 2 and 3; whether an entry is K or V is
  // uniform over a wave because KCH is a multiple of 64).
  constexpr int KCH = KT * (KD / 8);
  static_assert((2 * KCH) % NT == 0, "the chunk list divides evenly");
  constexpr int NL = 2 * KCH / NT;
  u32x4 rc[NL];
  bool row_ok[NL];
  float rkm = 1.f, rkp = 1.f;  // key mask / key padding flag of key tid (threads 0..63)
  const int bb = a.bias_mod > 0 ? b % a.bias_mod : b;  // batch index of bias / padding masks
  const int* krows = a.key_rows ? a.key_rows + (int64_t)bb * a.Sk : nullptr;
  const float* kmask = a.key_mask ? a.key_mask + (int64_t)b * a.km_sb : nullptr;
  const float* kpad = a.kpad ? a.kpad + (int64_t)bb * a.kp_sb : nullptr;
  int k0_loaded = 0;
  // entry i of this thread: chunk e (K) or e - KCH (V) of its tile, key = chunk / (KD/8), c = chunk % (KD/8)
  bool is_v[NL];
  int ch_key[NL], ch_c[NL];
  // FAST: byte offset of the chunk from the first key row of a tile (the launcher has checked that 64 rows
  // of K or V span less than 2 GB)
  uint32_t choff[NL];
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int e = tid + i * NT;
    is_v[i] = e >= KCH;
    const int ch = is_v[i] ? e - KCH : e;
    ch_key[i] = ch / (KD / 8);
    ch_c[i] = ch % (KD / 8);
    choff[i] = (uint32_t)(ch_key[i] * (is_v[i] ? a.v_ss : a.k_ss) + (ch_c[i] < dch ? ch_c[i] : 0) * 8) * 2u;
  }
  // Rows of the chunks this thread moves.  With key_rows they are looked
  // up one tile before the chunks themselves are requested, so that a tile
  // costs one memory round trip, not two in a row.
  int row_i[NL];
  auto gidx = [&](int k0) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int key = min(k0 + ch_key[i], a.Sk - 1);
      row_i[i] = krows ? krows[key] : key;
    }
  };
  auto gload = [&](int k0) {
    k0_loaded = k0;
    if (FAST && k0 + KT <= a.Sk) {  // (workgroup-uniform)
      const char* kb = reinterpret_cast<const char*>(kg + (int64_t)k0 * a.k_ss);
      const char* vb = reinterpret_cast<const char*>(vg + (int64_t)k0 * a.v_ss);
#pragma unroll
      for (int i = 0; i < NL; ++i) rc[i] = *reinterpret_cast<const u32x4*>((is_v[i] ? vb : kb) + choff[i]);
    } else {
      if constexpr (FAST) gidx(k0);
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const int row = row_i[i];
        row_ok[i] = row >= 0;
        rc[i] = *reinterpret_cast<const u32x4*>((is_v[i] ? vg : kg) + (int64_t)max(row, 0) * (is_v[i] ? a.v_ss : a.k_ss) +
                                                (ch_c[i] < dch ? ch_c[i] : 0) * 8);
      }
    }
    if (tid < KT) {
      const int key = min(k0 + tid, a.Sk - 1);
      if (kmask) rkm = kmask[key];
      if (kpad) rkp = kpad[key];
    }
  };
  auto sstore = [&](int buf) {
    const u32x4 z = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int key = ch_key[i], c = ch_c[i];
      const bool ok = k0_loaded + key < a.Sk && c < dch && (FAST || row_ok[i]);  // (FAST: rows are never negative)
      const u32x4 vv = ok ? rc[i] : z;
      if (!is_v[i]) *reinterpret_cast<u32x4*>(&sK[buf][key * LDK + c * 8]) = vv;
      else *reinterpret_cast<u32x4*>(&sV[buf][key * LDV + c * 8]) = vv;
    }
    if (tid < KT) {  // wave 0, all of it (KT = 64)
      const int code = (k0_loaded + tid >= a.Sk ? KEY_BEYOND : 0) | (rkm == 0.f ? KEY_MASKED : 0) | (rkp == 0.f ? KEY_PAD : 0);
      sCode[buf][tid] = code;
      const bool any = __any(code != 0);
      if (tid == 0) sAnyCode[buf] = any ? 1 : 0;
    }
  };
  // V columns that no chunk covers (head dimension padding: columns KD .. 32 DVT - 1 of either buffer) must
  // read as zero
  if constexpr (KD < DVT * 32) {
    constexpr int PAD = DVT * 32 - KD;  // a multiple of 16
    for (int idx = tid; idx < 2 * KT * (PAD / 2); idx += NT) {
      const int row = idx / (PAD / 2), w = idx % (PAD / 2);
      reinterpret_cast<uint32_t*>(&sV[row / KT][(row % KT) * LDV + KD])[w] = 0u;
    }
  }  // (no tile store touches these columns; the barrier after the first tile's stores orders them too)

  f32x16 o[DVT];
#pragma unroll
  for (int t = 0; t < DVT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[t][r] = 0.f;
  float m_run = NEG_INF, l_run = 0.f;  // softmax base (a maximum seen so far) in natural units, and row sum

  // Pair bias (fp32, one row per query): the 8 quads of a 64-key tile are
  // fetched one tile ahead, unconditionally, from addresses clamped into the
  // row (a clamped quad belongs to keys >= Sk, which are masked anyway).
  const float* bias_plane = a.bias ? a.bias + (int64_t)bb * a.bias_sb + (int64_t)h * a.bias_sh : nullptr;  // (uniform)
  const float* bias_row = a.bias ? bias_plane + (int64_t)qi * a.bias_sq : nullptr;
  const bool q_is_pad = a.qpad ? (a.qpad[(int64_t)bb * a.qp_sb + qi] == 0.f) : false;
  const bool bias_vec = FAST || (a.bias && a.Sk >= 4 && ((a.bias_sq & 3) == 0) && ((a.bias_sb & 3) == 0) &&
                                 ((a.bias_sh & 3) == 0) && ((a.bias_squad & 3) == 0) && (((uintptr_t)a.bias & 15) == 0));
  // key k of the row: at k (row-major) or, with quads of four keys as the outer
  // index, at (k / 4) * bias_squad + k % 4
  const int64_t quad_step = a.bias_squad ? a.bias_squad : 4;
  const int last_quad = (a.Sk - 1) & ~3;
  // FAST: this lane's byte offset from the tile's first quad of the bias plane (checked by the launcher to fit)
  const uint32_t bias_lane = (uint32_t)((int64_t)qi * a.bias_sq + hh * quad_step) * 4u;
  // the quads of tile k0 into `dst`, laid out like the score accumulators:
  // dst[u][4g + e] = bias(query, key k0 + 32u + 8g + 4hh + e)
  // `part` < 0: all eight quads; 0..3: the two quads (u = part / 2, g = 2 (part % 2) + {0, 1}) only
  auto gload_bias = [&](f32x16 (&dst)[2], int k0, int part = -1) {
    if (!bias_vec) return;  // workgroup-uniform
    const bool fast_addr = FAST && k0 + KT <= a.Sk;
    const char* bt = reinterpret_cast<const char*>(bias_plane + (int64_t)(k0 >> 2) * quad_step);
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        if (part >= 0 && (u != (part >> 1) || (g >> 1) != (part & 1))) continue;
        f32x4 v;
        if (fast_addr) v = *reinterpret_cast<const f32x4*>(bt + (int64_t)(8 * u + 2 * g) * quad_step * 4 + bias_lane);
        else v = *reinterpret_cast<const f32x4*>(bias_row + (int64_t)(min(k0 + u * 32 + 8 * g + 4 * hh, last_quad) >> 2) * quad_step);
        dst[u][4 * g] = v.x; dst[u][4 * g + 1] = v.y; dst[u][4 * g + 2] = v.z; dst[u][4 * g + 3] = v.w;
      }
  };

  const int nkt = (a.Sk + KT - 1) / KT;
  // Two register sets of 2 x 16 values.  FAST: they alternate between the tiles, the set of tile kt + 1
  // receives that tile's bias while tile kt is worked on and is then accumulated on by the matrix unit.
  // Otherwise one set holds the scores and the other the prefetched bias, copied over before the products.
  f32x16 setA[2], setB[2];
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int r = 0; r < 16; ++r) setA[u][r] = setB[u][r] = 0.f;
  if constexpr (!FAST) gidx(0);
  gload(0);
  if constexpr (!FAST) gidx(KT);
  gload_bias(FAST ? setA : setB, 0);
  // the output gate of the lane's query: asked for now, used after the last tile
  u32x2 gate_w[DVT][4];
#pragma unroll
  for (int t = 0; t < DVT; ++t)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int dd = 32 * t + 8 * g + 4 * hh;
      gate_w[t][g] = u32x2{0x3F803F80u, 0x3F803F80u};
      if (a.g) gate_w[t][g] = *reinterpret_cast<const u32x2*>(a.g + (int64_t)b * a.g_sb + (int64_t)qi * a.g_ss + h * d + (dd < d ? dd : 0));
    }
  sstore(0);
  lds_barrier();

  // One key tile.  FAST: `s` holds the tile's bias, `other` takes the next tile's.  Otherwise `other`
  // holds this tile's bias, is copied to `s`, and then takes the next tile's.
  auto tile = [&](int kt, f32x16 (&s)[2], f32x16 (&other)[2]) {
    const int buf = kt & 1;
    const int k0 = kt * KT;
    // next tile's K / V chunks (their rows are known) and the rows of the one after
    gload((kt + 1) * KT);
    if constexpr (!FAST) gidx((kt + 2) * KT);
    // FAST: the next tile's bias is requested in four pieces spread over this tile (below).  A wave that
    // issues a burst of loads sits at them until the CU's address unit, which takes 16 to 64 cycles per wave
    // instruction and serves eight waves, has accepted them all; spread out, the unit works through them
    // while the wave computes.
    auto bias_piece = [&](int part) {
      if constexpr (FAST) {
        __builtin_amdgcn_sched_barrier(0);
        gload_bias(other, (kt + 1) * KT, part);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // both 32-key halves through the matrix unit first (two independent chains);
    // s[u][4g + e] = logit(query j, key k0 + 32u + 8g + 4hh + e)
    // (either form starts the accumulation from the bias, so both give the same bits)
    if constexpr (!FAST) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float bv = 0.f;
            if (bias_vec) bv = other[u][4 * g + e];
            else if (bias_row) {
              const int kc = min(k0 + u * 32 + 8 * g + 4 * hh + e, a.Sk - 1);
              bv = bias_row[(int64_t)(kc >> 2) * quad_step + (kc & 3)];
            }
            s[u][4 * g + e] = bv;
          }
      gload_bias(other, (kt + 1) * KT);  // the next tile's bias into the registers just read
    }
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
        s[u] = mfma32(lds_frag(sK[buf], LDK, u * 32, ks * 16, lane), qf[ks], s[u]);
    bias_piece(0);
    // Masks from the per-key codes; most tiles carry none (a workgroup-uniform
    // test skips the block).  The logits stay in natural units: the maximum
    // does not care, and exp2 takes fma(s, log2 e, -m log2 e).  (For a row
    // whose keys are all masked every s equals m = -1e9 and the fma leaves the
    // rounding error of m log2 e, at most 2^6 in magnitude and the same for
    // every key: the weights stay uniform.)
    if (__builtin_amdgcn_readfirstlane(sAnyCode[buf])) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int* cp = &sCode[buf][u * 32 + 8 * g + 4 * hh];
          const int code[4] = {cp[0], cp[1], cp[2], cp[3]};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float v = s[u][4 * g + e];
            if (code[e] & KEY_MASKED) v = -1e9f;
            if (q_is_pad && (code[e] & KEY_PAD)) v += 1e9f;
            if (code[e] & KEY_BEYOND) v = NEG_INF;
            s[u][4 * g + e] = v;
          }
        }
    }
    // maximum of the lane's 32 logits as a tree of three-input maxima
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
    bias_piece(1);
    // The base of the exponentials follows the maximum lazily: it moves only when a tile's maximum
    // exceeds it by more than BASE_SLACK (weights then reach e^BASE_SLACK at most, far inside fp32 and
    // bf16 range; the normalisation at the end takes the common factor out again), so that most tiles
    // leave the output accumulators alone.  The first tile moves it from -inf to its maximum.
    constexpr float BASE_SLACK = 8.f;
    const float m_new = mx - m_run > BASE_SLACK ? mx : m_run;
    const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * LOG2E);  // 0 on the first tile (m_run = -inf, m_new finite)
    m_run = m_new;
    const float m2 = m_new * LOG2E;
    bf16x8 pf[2][2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        float pv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) pv[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[u][8 * half + e], LOG2E, -m2));
        pf[u][half] = as_frag(pack8(pv));
        if (half == 1) bias_piece(2 + u);
      }
    // row sums of the ROUNDED probabilities on the matrix unit (ones * P), so
    // that the weights that multiply V sum to exactly one after normalisation
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
      for (int t = 0; t < DVT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[t][r] *= alpha;
    }
    // O^T[dd][query] += sum_key V^T[dd][key] P^T[key][query]; fragment element e
    // of lane-half hh in k-step `half` is key 32u + 16*half + 8*(e>>2) + 4*hh + (e&3).  V lies in LDS as it
    // lies in memory, [key][dd]; the transposing LDS read hands each lane of a group of 16 one column of a
    // 4-row x 16-column block (lane i of the group points at row i / 4, columns 4 (i % 4) .. of the block
    // and receives column i of its four rows): rows = four consecutive keys, columns = the group's 16 dd.
    {
      const int i16 = lane & 15;
      const bf16_t* vbase = &sV[buf][(4 * hh + (i16 >> 2)) * LDV + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3)];
#pragma unroll
      for (int t = 0; t < DVT; ++t)
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const bf16_t* vp = vbase + (u * 32 + 16 * half) * LDV + t * 32;
            const v4s lo = lds_read_tr16(vp), hi = lds_read_tr16(vp + 8 * LDV);
            o[t] = mfma32(as_frag(__builtin_bit_cast(u32x4, v8s{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w})),
                          pf[u][half], o[t]);
          }
    }
    if (kt + 1 < nkt) sstore(buf ^ 1);
    lds_barrier();
  };
  if constexpr (FAST) {
    for (int kt = 0; kt < nkt; kt += 2) {
      tile(kt, setA, setB);
      if (kt + 1 < nkt) tile(kt + 1, setB, setA);
    }
  } else {
    for (int kt = 0; kt < nkt; ++kt) tile(kt, setA, setB);
  }

  const float inv = 1.f / l_run;  // the ones * P sums cover both half-waves' keys
  if (!q_ok) return;
  // o[t][4g + e] = out(query j, head-dim 32t + 8g + 4hh + e)
#pragma unroll
  for (int t = 0; t < DVT; ++t)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int dd = 32 * t + 8 * g + 4 * hh;
      if (dd >= d) continue;  // d % 4 == 0, so a quad is all in or all out
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = o[t][4 * g + e] * inv;
      {
        const u32x2 gw = gate_w[t][g];   // ones without a gate
        v[0] *= bflo(gw.x); v[1] *= bfhi(gw.x); v[2] *= bflo(gw.y); v[3] *= bfhi(gw.y);
      }
      const int64_t off = (int64_t)b * a.o_sb + (int64_t)qi * a.o_ss + h * d + dd;
      if (a.out_f32) {
        f32x4 w = {v[0], v[1], v[2], v[3]};
        *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(a.out) + off) = w;
      } else {
        u32x2 w;
        w.x = pack2bf(v[0], v[1]);
        w.y = pack2bf(v[2], v[3]);
        *reinterpret_cast<u32x2*>(reinterpret_cast<bf16_t*>(a.out) + off) = w;
      }
    }
}

// Queries per workgroup: 128 (four waves share the K / V tiles), or 64 when
// that would leave the 256 CUs with too few workgroups, or 32 for the short
// query windows of the atom cross-attention.
template <int KSTEPS, int DVT>
int launch_nw(const FlashArgs& a, hipStream_t stream) {
  const int64_t heads = (int64_t)a.H * a.B;
  // Four waves share each staged K / V tile once there are enough 128-query
  // workgroups to cover the chip; below that, two waves per workgroup spread
  // the work over twice as many CUs.
  const int nw = a.Sq <= 32 ? 1 : (((a.Sq + 127) / 128) * heads < 256 ? 2 : 4);
  const int64_t n_blocks = (int64_t)((a.Sq + nw * 32 - 1) / (nw * 32)) * heads;
  if (n_blocks <= 0 || n_blocks > 0x7ffffff0) return AF3_ERR_BAD_ARG;
  FlashArgs fa = a;
  fa.n_blocks = (int)n_blocks;
  const dim3 grid((unsigned)((n_blocks + 7) / 8 * 8));  // whole rounds over the 8 XCDs; the surplus ids return at once
  // The form with fixed per-lane offsets: no row table, a bias that can be fetched 16 bytes at a time, and
  // offsets inside a key tile / a bias plane that fit 32 bits.
  const int64_t quad_step = a.bias_squad ? a.bias_squad : 4;
  const bool fast = !a.key_rows && a.bias && a.Sk >= 4 && (a.bias_sq & 3) == 0 && (a.bias_sb & 3) == 0 &&
                    (a.bias_sh & 3) == 0 && (a.bias_squad & 3) == 0 && ((uintptr_t)a.bias & 15) == 0 &&
                    a.k_ss > 0 && a.v_ss > 0 && a.k_ss < (1 << 22) && a.v_ss < (1 << 22) && a.bias_sq >= 0 &&
                    quad_step > 0 && (int64_t)a.Sq * a.bias_sq + quad_step < (1 << 28);
  // (with a single wave, or with head dimension 48 and fewer than four waves, to share the K / V staging
  // registers between, the second register set of that form no longer fits: those take the general form)
#define AF3_FLASH_LAUNCH(NW_)                                                                                   \
  do {                                                                                                          \
    if constexpr (NW_ == 4 || (KSTEPS < 3 && NW_ == 2)) {                                                       \
      if (fast) {                                                                                               \
        hipLaunchKernelGGL((flash_kernel<KSTEPS, DVT, NW_, true>), grid, dim3(NW_ * 64), 0, stream, fa);        \
        break;                                                                                                  \
      }                                                                                                         \
    }                                                                                                           \
    hipLaunchKernelGGL((flash_kernel<KSTEPS, DVT, NW_, false>), grid, dim3(NW_ * 64), 0, stream, fa);           \
  } while (0)
  if (nw == 1) AF3_FLASH_LAUNCH(1);
  else if (nw == 2) AF3_FLASH_LAUNCH(2);
  else AF3_FLASH_LAUNCH(4);
#undef AF3_FLASH_LAUNCH
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

}  // namespace

int launch_flash_attention(const FlashArgs& a, hipStream_t stream) {
  if (a.B <= 0 || a.H <= 0 || a.Sq <= 0 || a.Sk <= 0 || !a.q || !a.k || !a.v || !a.out) return AF3_ERR_BAD_ARG;
  if (a.d != 16 && a.d != 24 && a.d != 32 && a.d != 48) return AF3_ERR_UNSUPPORTED;
  const int64_t strides[] = {a.q_sb, a.q_ss, a.k_sb, a.k_ss, a.v_sb, a.v_ss, a.g_sb, a.g_ss, a.o_sb, a.o_ss};
  for (int64_t s : strides)
    if (s & 7) return AF3_ERR_BAD_ARG;
  if (((uintptr_t)a.q & 15) || ((uintptr_t)a.k & 15) || ((uintptr_t)a.v & 15) || ((uintptr_t)a.g & 15) ||
      ((uintptr_t)a.out & 15))
    return AF3_ERR_BAD_ARG;
  if ((a.qpad == nullptr) != (a.kpad == nullptr)) return AF3_ERR_BAD_ARG;
  if (a.bias_mod < 0 || (a.bias_mod > 0 && a.B % a.bias_mod) || (a.key_rows && a.bias_mod <= 0)) return AF3_ERR_BAD_ARG;
  if (a.bias_squad && (a.bias_sq != 4 || (a.bias_squad & 3))) return AF3_ERR_BAD_ARG;
  if (a.d == 48) return launch_nw<3, 2>(a, stream);
  if (a.d == 16) return launch_nw<1, 1>(a, stream);
  return launch_nw<2, 1>(a, stream);
}
