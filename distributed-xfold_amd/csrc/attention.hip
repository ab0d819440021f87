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
// fragment uses the same order).  K and V^T tiles of 64 keys are staged in LDS,
// double-buffered, and shared by the workgroup's waves.
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
constexpr int LDV = KT + 8;   // sVt row stride (bf16)
constexpr float NEG_INF = -__builtin_huge_valf();

template <int KSTEPS, int DVT, int NW>
__global__ __launch_bounds__(NW * 64) void flash_kernel(FlashArgs a) {
  constexpr int KD = KSTEPS * 16;  // padded q/k head dim
  constexpr int LDK = KD + 8;      // sK row stride (bf16)
  constexpr int NT = NW * 64;
  __shared__ __attribute__((aligned(16))) bf16_t sK[2][KT * LDK];
  __shared__ __attribute__((aligned(16))) bf16_t sVt[2][DVT * 32 * LDV];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hh = lane >> 5, j = lane & 31;
  const int xaddr = half_swap_addr();
  // blockIdx.x = (q_tile * H + head) * B + batch: workgroups in flight together
  // share one (head, q-tile) slab of the pair bias across many batch rows.
  const int b = blockIdx.x % a.B;
  const int h = (blockIdx.x / a.B) % a.H;
  const int q0 = (blockIdx.x / (a.B * a.H)) * (NW * 32) + wave * 32;
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
      u32x4 v = {0, 0, 0, 0};
      if (c < d) v = *reinterpret_cast<const u32x4*>(qp + c);
      qf[ks] = as_frag(v);
    }
  }

  const bf16_t* kg = a.k + (int64_t)b * a.k_sb + h * d;
  const bf16_t* vg = a.v + (int64_t)b * a.v_sb + h * d;
  const int dch = d / 8;  // 16-byte chunks per real key row

  // tile loaders (global -> registers -> LDS), chunk id = key * (KD/8) + c
  constexpr int KCH = KT * (KD / 8);
  constexpr int NLD = (KCH + NT - 1) / NT;
  u32x4 rk[NLD], rv[NLD];
  auto gload = [&](int k0) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int idx = tid + i * NT;
      const int key = idx / (KD / 8), c = idx % (KD / 8);
      const u32x4 z = {0, 0, 0, 0};
      rk[i] = z; rv[i] = z;
      if (idx < KCH && k0 + key < a.Sk && c < dch) {
        rk[i] = *reinterpret_cast<const u32x4*>(kg + (int64_t)(k0 + key) * a.k_ss + c * 8);
        rv[i] = *reinterpret_cast<const u32x4*>(vg + (int64_t)(k0 + key) * a.v_ss + c * 8);
      }
    }
  };
  auto sstore = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int idx = tid + i * NT;
      if (idx >= KCH) continue;
      const int key = idx / (KD / 8), c = idx % (KD / 8);
      *reinterpret_cast<u32x4*>(&sK[buf][key * LDK + c * 8]) = rk[i];
      if (c * 8 < DVT * 32) {
        const uint32_t w4[4] = {rv[i].x, rv[i].y, rv[i].z, rv[i].w};
#pragma unroll
        for (int e = 0; e < 8; ++e)
          sVt[buf][(c * 8 + e) * LDV + key] = (bf16_t)((e & 1) ? (w4[e >> 1] >> 16) : (w4[e >> 1] & 0xffffu));
      }
    }
  };
  // V^T rows that no chunk covers (head dim padding) must read as zero
  for (int idx = tid; idx < 2 * DVT * 32 * LDV; idx += NT) (&sVt[0][0])[idx] = 0;
  lds_barrier();

  f32x16 o[DVT];
#pragma unroll
  for (int t = 0; t < DVT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[t][r] = 0.f;
  float m_run = NEG_INF, l_run = 0.f;

  const int bb = a.bias_mod > 0 ? b % a.bias_mod : b;  // batch index of bias / padding masks
  const float* bias_row = a.bias ? a.bias + (int64_t)bb * a.bias_sb + (int64_t)h * a.bias_sh + (int64_t)qi * a.bias_sq : nullptr;
  const float* kmask = a.key_mask ? a.key_mask + (int64_t)b * a.km_sb : nullptr;
  const float* kpad = a.kpad ? a.kpad + (int64_t)bb * a.kp_sb : nullptr;
  const bool q_is_pad = a.qpad ? (a.qpad[(int64_t)bb * a.qp_sb + qi] == 0.f) : false;
  const bool bias_vec = a.bias && ((a.bias_sq & 3) == 0) && ((a.bias_sb & 3) == 0) && ((a.bias_sh & 3) == 0) &&
                        (((uintptr_t)a.bias & 15) == 0);

  const int nkt = (a.Sk + KT - 1) / KT;
  gload(0);
  sstore(0);
  lds_barrier();

  for (int kt = 0; kt < nkt; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nkt) gload((kt + 1) * KT);
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const int kbase = kt * KT + sub * 32;
      if (kbase >= a.Sk) break;  // uniform across the workgroup
      f32x16 s;
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
        s = mfma32(lds_frag(sK[buf], LDK, sub * 32, ks * 16, lane), qf[ks], s);
      // s[4g + e] = logit(query j, key kbase + 8g + 4hh + e)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int key0 = kbase + 8 * g + 4 * hh;
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (bias_row) {
          if (bias_vec && key0 + 3 < a.Sk) {
            const f32x4 t4 = *reinterpret_cast<const f32x4*>(bias_row + key0);
            bv[0] = t4.x; bv[1] = t4.y; bv[2] = t4.z; bv[3] = t4.w;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (key0 + e < a.Sk) bv[e] = bias_row[key0 + e];
          }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int key = key0 + e;
          float v = s[4 * g + e] + bv[e];
          if (key >= a.Sk) {
            v = NEG_INF;
          } else {
            if (kmask && kmask[key] == 0.f) v = -1e9f;
            if (q_is_pad && kpad[key] == 0.f) v += 1e9f;
          }
          s[4 * g + e] = v;
        }
      }
      float mx = s[0];
#pragma unroll
      for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s[r]);
      mx = fmaxf(mx, half_swap(xaddr, mx));
      const float m_new = fmaxf(m_run, mx);
      const float alpha = __expf(m_run - m_new);  // 0 on the first tile (m_run = -inf, m_new finite)
      m_run = m_new;
      float psum = 0.f;
      bf16x8 pf[2];
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        float pv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) pv[e] = __expf(s[8 * half + e] - m_new);
        const u32x4 pk = pack8(pv);
        // the row sum uses the rounded probabilities so that the weights that
        // multiply V sum to exactly one after normalisation
        float back[8];
        unpack8(pk, back);
#pragma unroll
        for (int e = 0; e < 8; ++e) psum += back[e];
        pf[half] = as_frag(pk);
      }
      l_run = l_run * alpha + psum;
      if (__any(alpha != 1.f)) {
#pragma unroll
        for (int t = 0; t < DVT; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[t][r] *= alpha;
      }
      // O^T[dd][query] += sum_key V^T[dd][key] P^T[key][query]; fragment element e
      // of lane-half hh in k-step `half` is key kbase + 16*half + 8*(e>>2) + 4*hh + (e&3)
#pragma unroll
      for (int t = 0; t < DVT; ++t)
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const bf16_t* vp = &sVt[buf][(t * 32 + j) * LDV + sub * 32 + 16 * half + 4 * hh];
          const u32x2 lo = *reinterpret_cast<const u32x2*>(vp);
          const u32x2 hi = *reinterpret_cast<const u32x2*>(vp + 8);
          u32x4 vv;
          vv.x = lo.x; vv.y = lo.y; vv.z = hi.x; vv.w = hi.y;
          o[t] = mfma32(as_frag(vv), pf[half], o[t]);
        }
    }
    if (kt + 1 < nkt) sstore(buf ^ 1);
    lds_barrier();
  }

  const float l_tot = l_run + half_swap(xaddr, l_run);
  const float inv = 1.f / l_tot;
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
      if (a.g) {
        const u32x2 gw = *reinterpret_cast<const u32x2*>(a.g + (int64_t)b * a.g_sb + (int64_t)qi * a.g_ss + h * d + dd);
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

template <int KSTEPS, int DVT>
int launch_nw(const FlashArgs& a, hipStream_t stream) {
  const bool small = a.Sq <= 32;
  const int qper = small ? 32 : 128;
  const int64_t blocks = (int64_t)((a.Sq + qper - 1) / qper) * a.H * a.B;
  if (blocks <= 0 || blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  if (small) hipLaunchKernelGGL((flash_kernel<KSTEPS, DVT, 1>), dim3((unsigned)blocks), dim3(64), 0, stream, a);
  else hipLaunchKernelGGL((flash_kernel<KSTEPS, DVT, 4>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

}  // namespace

int launch_flash_attention(const FlashArgs& a, hipStream_t stream) {
  if (a.B <= 0 || a.H <= 0 || a.Sq <= 0 || a.Sk <= 0 || !a.q || !a.k || !a.v || !a.out) return AF3_ERR_BAD_ARG;
  if (a.d != 24 && a.d != 32 && a.d != 48) return AF3_ERR_UNSUPPORTED;
  const int64_t strides[] = {a.q_sb, a.q_ss, a.k_sb, a.k_ss, a.v_sb, a.v_ss, a.g_sb, a.g_ss, a.o_sb, a.o_ss};
  for (int64_t s : strides)
    if (s & 7) return AF3_ERR_BAD_ARG;
  if (((uintptr_t)a.q & 15) || ((uintptr_t)a.k & 15) || ((uintptr_t)a.v & 15) || ((uintptr_t)a.g & 15) ||
      ((uintptr_t)a.out & 15))
    return AF3_ERR_BAD_ARG;
  if ((a.qpad == nullptr) != (a.kpad == nullptr)) return AF3_ERR_BAD_ARG;
  if (a.d == 48) return launch_nw<3, 2>(a, stream);
  return launch_nw<2, 1>(a, stream);
}
