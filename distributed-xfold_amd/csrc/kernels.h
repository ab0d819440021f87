// Host-side launch interface of the kernels (internal; the public C ABI is in
// include/af3_hip.h and implemented in api.hip).
#pragma once
#include "common.h"

// ------------------------------------------------------------------ gemm.hip
enum { EPI_PLAIN = 0, EPI_SEGMENTED = 1, EPI_SWIGLU = 2, EPI_GATE_RES = 3 };
enum { SEG_PLAIN = 0, SEG_BIAS_SCALE = 1, SEG_SIGMOID = 2 };

struct GemmArgs {
  const bf16_t* A = nullptr;  // [batch][M][lda]
  const bf16_t* B = nullptr;  // [batch][N][ldb]   (C = A * B^T)
  void* C = nullptr;          // [batch][M][ldc]   bf16 or fp32
  int M = 0, N = 0, K = 0, batch = 1;
  int64_t lda = 0, ldb = 0, ldc = 0, sA = 0, sB = 0, sC = 0;
  int out_f32 = 0;
  int epi = EPI_PLAIN;
  float alpha = 1.f;            // PLAIN: (acc + bias) * alpha ; SEG_BIAS_SCALE likewise
  const float* bias = nullptr;  // indexed by output column: entries 0 .. bias_len - 1 exist
  int64_t bias_len = 0;         // a launch whose epilogue would read past it is refused (gemm_bias_span)
  int act_sigmoid = 0;          // PLAIN only
  int seg_len = 0, seg_ops = 0; // SEGMENTED: op of column segment s in bits [4s, 4s+4)
  const float* gate = nullptr;  // GATE_RES: multiply by gate[m % gate_rows][n]
  int gate_rows = 0;
  int gate_per_row = 0;         // GATE_RES: gate is one factor per row, gate[m % gate_rows]
  int64_t ld_gate = 0;
  const float* res_f32 = nullptr;   // GATE_RES: residual added last (either dtype)
  const bf16_t* res_bf16 = nullptr;
  int64_t ld_res = 0, sRes = 0;
  int vec_ok = 0, res_vec_ok = 0, gate_vec_ok = 0;  // set by launch_gemm_nt: rows aligned for 16-byte stores / loads
  // regroup32 (PLAIN, batch 1, M and N multiples of 32): element (m, n) is stored
  // at [(m / 32, n / 32)][(m % 32, n % 32)], i.e. C is [(M/32)(N/32)][1024]:
  // the outer products of 32-channel rows, one contiguous 1024-vector per pair.
  int regroup32 = 0;
};
int launch_gemm_nt(const GemmArgs& g, hipStream_t stream);
// Which bias entries a launch reads.  Column c takes bias[c] when the epilogue is not segmented, or
// when c lies in a segment whose op is SEG_BIAS_SCALE; the kernels read whole groups of entries
// (gemm_nt_kernel up to 8 from a multiple of 8, the large tile 4 from a multiple of 4, the last
// group pulled back to end at N).  The device code takes its addresses from these functions, the
// host takes the extent it checks against bias_len from them: one formula for both.
__host__ __device__ inline bool gemm_col_uses_bias(const GemmArgs& g, int col) {
  if (!g.bias) return false;
  if (g.epi != EPI_SEGMENTED) return true;
  return ((g.seg_ops >> (4 * (col / g.seg_len))) & 15) == SEG_BIAS_SCALE;
}
// large tile: the 4 entries a lane fetches for columns colb .. colb + 3 of its wave (colb may lie past N)
__host__ __device__ inline bool big_tile_bias_quad(const GemmArgs& g, int colb, int* first) {
  *first = (colb < g.N - 4 ? colb : g.N - 4);
  return gemm_col_uses_bias(g, colb < g.N - 1 ? colb : g.N - 1);
}
// Half-open range [first, last) of bias entries the launch of `g` reads (big: on the large tile);
// first == last: none.
void gemm_bias_span(const GemmArgs& g, bool big, int64_t* first, int64_t* last);
// contract.hip: the same product, plain bf16 output, 256x256 tiles (large M, N)
bool contract_supported(const GemmArgs& g);
int launch_contract(const GemmArgs& g, hipStream_t stream);
// the 256x256 tile with the epilogues of the dense projections (bias / scale /
// sigmoid per column segment, SwiGLU, regrouped output): big_tile_mode names the
// kernel instance that can take `g`, or -1
int big_tile_mode(const GemmArgs& g);
int launch_big_tile(const GemmArgs& g, int mode, hipStream_t stream);
// the large-tile instance launch_gemm_nt hands `g` to, or -1: the 128x128-tile kernel
int gemm_big_tile_choice(const GemmArgs& g);

// ---------------------------------------------------------------- rowops.hip
// y = LN(x) [* weight + bias] ; then, if scale: y = sigmoid(scale[r]) * y + shift[r]
// with r = row % cond_rows (conditioning shared by the sample batch).
struct RowNormArgs {
  const void* x = nullptr;  // [rows][ldx] bf16 or fp32
  int x_f32 = 0;
  bf16_t* y = nullptr;      // [rows][ldy]
  int64_t rows = 0, ldx = 0, ldy = 0;
  int C = 0;
  const float* weight = nullptr;  // [C] or null
  const float* bias = nullptr;    // [C] or null
  const float* scale = nullptr;   // [cond_rows][ld_cond] pre-sigmoid, or null
  const float* shift = nullptr;
  int64_t cond_rows = 0, ld_cond = 0;
  int param_vec = 0, cond_vec = 0;  // set by launch_row_norm: arrays aligned for 16-byte loads
};
int launch_row_norm(const RowNormArgs& a, hipStream_t stream);
// out[c][r] = in[r][c], bf16, rows and cols multiples of 8
// out[b][t][:] = sum over slots a, idx[t][a] >= 0, of relu(src[b][idx[t][a]][:]) / count[t]  (fp32 out, <= 32 slots)
int launch_gathered_relu_mean(const bf16_t* src, const int* idx, const float* count, float* out, int64_t batch,
                              int64_t n_src, int64_t n_out, int slots, int channels, hipStream_t stream);
// out[b][q][:] = cond[q][:] + w pos[b][rows[q]]  (3 coordinates -> channels; rows[q] < 0: cond only)
int launch_atom_position_features(const float* pos, const int* rows, const float* w, const float* cond, void* out,
                                  int out_f32, int64_t batch, int64_t n_slots, int64_t n_q, int channels,
                                  hipStream_t stream);
// out[b][q][:] = (rows[q] >= 0 ? src[b][rows[q]][:] : 0) + add[b][q][:]   (all bf16)
int launch_gather_rows_add(const bf16_t* src, const int* rows, const bf16_t* add, bf16_t* out, int64_t batch,
                           int64_t n_src, int64_t n_q, int channels, hipStream_t stream);
// out[b][t][0..2] = w LayerNorm(x[b][rows[t]]) * ln_w  (rows[t] < 0: zeros); channels = 128, fp32 out
int launch_ln_project3_gather(const bf16_t* x, const int* rows, const float* ln_w, const float* w, float* out,
                              int64_t batch, int64_t n_src, int64_t n_out, int channels, hipStream_t stream);
int launch_transpose(const bf16_t* in, bf16_t* out, int64_t rows, int64_t cols, hipStream_t stream);
// y[r][k] = softmax_k(x[r][k] + 1e9 (mask[k] - 1)) as bf16, x [rows][cols] fp32, y rows ldy apart (the tail zero)
int launch_softmax_rows(const float* x, const float* mask, bf16_t* y, int64_t rows, int cols, int64_t ldy,
                        hipStream_t stream);
// y[r][:] = (res ? res[r][:] : 0) + W relu?(x[r][:]), fp32, W [n_out][k], n_out 16 or 3, k % 4 == 0, k <= 128
int launch_narrow_linear_f32(const float* x, const float* w, const float* res, float* y, int64_t rows, int k, int n_out,
                             int relu_in, hipStream_t stream);
int launch_atom_pair_logits(const float* x, const float* ln_w, const float* w, float* out, int64_t n_groups, int64_t group,
                            int n_blocks, int n_head, hipStream_t stream);
int launch_atom_pair_cond(const float* row, const float* col, const float* tp, const int* tq, const int* tk, int n_tok,
                          const float* q_pos, const float* k_pos, const int* q_uid, const int* k_uid, const float* w_off,
                          const float* w_dist, const float* w_valid, const float* w1, const float* w2, const float* w3,
                          float* out, int64_t subsets, int queries, int keys, hipStream_t stream);

// -------------------------------------------------------------- pair_tile.hip
// Residual-stream tensors (`pair`, `out`, `x`) are bf16 or fp32 (io_f32).
// LayerNorm over fewer than 128 real channels: the tensor and the weights are zero-padded to 128 and the
// statistics are taken over `valid` channels (sums over all 128 are sums over the valid ones; the padded
// channels' share of the squared deviations, pad * mean^2, is taken out again).  valid = 128: pad = 0,
// the same arithmetic bit for bit.
struct LnWidth {
  float inv_c = 1.f / 128.f;  // 1 / valid channels
  float pad = 0.f;            // 128 - valid channels
};
inline LnWidth ln_width(int valid) {
  LnWidth w;
  w.inv_c = 1.f / (float)valid;
  w.pad = (float)(128 - valid);
  return w;
}

struct TriMulArgs {
  LnWidth lw;
  int valid_c = 128;  // hidden channels 0 .. valid_c - 1 are real: the others are never contracted and count as zero
  const void* pair = nullptr;   // [N][N][128]
  const float* mask = nullptr;  // [N][N] 0/1 or null
  void* out = nullptr;          // [N][N][128]; may alias pair when residual
  int io_f32 = 0, N = 0, Np = 0, outgoing = 1, residual = 0;
  const float *ln_in_w = nullptr, *ln_in_b = nullptr, *ln_c_w = nullptr, *ln_c_b = nullptr;
  const bf16_t* w_pg = nullptr;   // [4][128][128]: per chunk 64 projection rows + 64 gate rows
  const bf16_t* w_gl = nullptr;   // [128][128] gating_linear
  const bf16_t* w_out = nullptr;  // [128][128] output_projection
  bf16_t *a_buf = nullptr, *b_buf = nullptr;  // [128][N][Np] channel-major operands
  const bf16_t* t_buf = nullptr;              // [128][N][Np] contraction result
};
int launch_trimul_prologue(const TriMulArgs& a, hipStream_t s);
int launch_trimul_epilogue(const TriMulArgs& a, hipStream_t s);

struct AttnProjArgs {
  LnWidth lw;
  const void* pair = nullptr;  // [N][N][128]
  int io_f32 = 0, N = 0, transpose = 0;
  int skip_ln = 0;  // pair is already normalised
  const float *ln_w = nullptr, *ln_b = nullptr;
  const bf16_t* w_main = nullptr;  // [n_chunks][128][128]
  int n_chunks = 0, chunk_ops = 0; // SEG_* per chunk, 4 bits each
  float q_scale = 1.f;
  bf16_t* out_main = nullptr;      // [(b*N + s)][ld_main], chunk c at columns 128c..
  int64_t ld_main = 0;
  const bf16_t* w_bias = nullptr;  // [roundup(n_bias, 32)][128]
  int n_bias = 0;
  float* out_bias = nullptr;       // [n_bias][N][N] fp32, or
  bf16_t* out_bias_bf16 = nullptr; // [n_bias][N][ld_bias] bf16 (values times bias_scale)
  int64_t ld_bias = 0;
  float bias_scale = 1.f;
};
int launch_attn_proj(const AttnProjArgs& a, hipStream_t s);

// pair_cond = Linear(LayerNorm([pair | relative encoding of the token pair])) without the concatenated
// tensor (pair_tile.hip).  The relative encoding has n_rel = 4 max_rel_idx + 2 max_rel_chain + 7 one-hot
// channels; g_hot[h][o] = ln_w[128 + h] * W[o][128 + h] and g_sum[o] = sum_h g_hot[h][o].
struct PairCondInitArgs {
  const void* pair = nullptr;  // [N][N][128], fp32 or bf16
  int io_f32 = 1, N = 0;
  float in_scale = 1.f;        // the pair values are multiplied by this first
  const int *asym_id = nullptr, *residue_index = nullptr, *token_index = nullptr, *entity_id = nullptr, *sym_id = nullptr;  // [N]
  int max_rel_idx = 32, max_rel_chain = 2, n_rel = 139;
  const float* ln_w = nullptr;     // [128] LayerNorm weights of the pair channels
  const bf16_t* w_pair = nullptr;  // [128][128] projection weights of the pair channels
  const float* g_hot = nullptr;    // [n_rel][128]
  const float* g_sum = nullptr;    // [128]
  float* out = nullptr;            // [N][N][128] fp32
};
int launch_pair_cond_init(const PairCondInitArgs& a, hipStream_t s);

struct AttnOutArgs {
  LnWidth lw;
  const bf16_t* og = nullptr;  // [(b*N + s)][ld_og] attention output, normalised, not yet gated
  int64_t ld_og = 0;
  const bf16_t* w_gate = nullptr;  // [128][128] gating_query: the gate is sigmoid(LN(pair) w_gate^T)
  const bf16_t* w_out = nullptr;   // [128][128]
  const void* pair = nullptr;      // gate input and residual source
  int skip_ln = 0;                 // pair is already normalised
  const float *ln_w = nullptr, *ln_b = nullptr;
  void* out = nullptr;
  int io_f32 = 0, N = 0, transpose = 0, residual = 0;
};
int launch_attn_out(const AttnOutArgs& a, hipStream_t s);

struct TransitionArgs {
  LnWidth lw;
  const void* x = nullptr;  // [N][128]
  void* out = nullptr;
  int io_f32 = 0, N = 0, hidden = 0, residual = 0;
  const float *ln_w = nullptr, *ln_b = nullptr;
  const bf16_t* w1 = nullptr;  // [hidden/64][128][128]: 64 a rows then 64 b rows per slab
  const bf16_t* w2 = nullptr;  // [128][hidden]
};
int launch_transition(const TransitionArgs& a, hipStream_t s);

// -------------------------------------------------------------- attention.hip
// q/k/v/g/out are addressed as base + batch * sb + position * ss + head * d.
struct FlashArgs {
  const bf16_t *q = nullptr, *k = nullptr, *v = nullptr, *g = nullptr;  // g: output gate or null
  int64_t q_sb = 0, q_ss = 0, k_sb = 0, k_ss = 0, v_sb = 0, v_ss = 0, g_sb = 0, g_ss = 0;
  void* out = nullptr;
  int out_f32 = 0;
  int64_t o_sb = 0, o_ss = 0;
  int B = 0, H = 0, Sq = 0, Sk = 0, d = 0;
  const float* bias = nullptr;  // [.][H][Sq][Sk], key stride 1
  int64_t bias_sb = 0, bias_sh = 0, bias_sq = 0;
  // bias_squad != 0: quads of four keys are the outer index, [.][H][Sk/4][Sq][4]:
  // key k of query q at q * bias_sq + (k / 4) * bias_squad + k % 4 with bias_sq = 4.
  // The lanes of a wave hold 32 consecutive queries, so a load of one quad per
  // lane is then one contiguous 512-byte run instead of 32 pieces of 16 bytes.
  int64_t bias_squad = 0;
  const float* key_mask = nullptr;  // [B][Sk] (km_sb may be 0): 0 -> logit replaced by -1e9
  int64_t km_sb = 0;
  const float *qpad = nullptr, *kpad = nullptr;  // [B][Sq], [B][Sk]: +1e9 where both are 0
  int64_t qp_sb = 0, kp_sb = 0;
  int bias_mod = 0;  // > 0: bias, qpad and kpad are indexed by batch % bias_mod
  // Gathered keys: key s of batch entry b is row key_rows[(b % bias_mod) * Sk + s]
  // of the K / V table of sample b / bias_mod (k_sb / v_sb: table stride); a
  // negative row is a key with zero K and V.  Null: key s is row s of batch b.
  const int* key_rows = nullptr;
  int n_blocks = 0;  // workgroups that have work (set by the launcher; the grid is rounded up to a multiple of 8)
};
int launch_flash_attention(const FlashArgs& a, hipStream_t stream);

// ------------------------------------------- triattn.hip, triattn_core.hip
// Scratch of the triangle-attention fast path, in the frame of the (possibly
// transposed) operator, rows b:
//   q, k     bf16 [b][h][s][32]   (q times log2(e)/sqrt(32))
//   vt       bf16 [b][h][32][ldn] V transposed, ldn = N rounded up to 16, columns >= N zero,
//            key k of a row stored at column tri_vt_pos(k): inside every aligned group of 16
//            keys the two middle quads are swapped, which makes the 8 keys one lane feeds to
//            a P.V MFMA (k, k+1, k+2, k+3, k+8, ..., k+11 with k % 8 == 0 or 4) 16 contiguous bytes
//   bias     fp16, pair bias times log2(e) (clamped to the fp16 range), in MFMA-fragment order:
//            the attention core adds it to the scores on the matrix unit, S^T += I * bias^T with an
//            fp16 identity, and wants per (head, 32-query block, 64-key tile) the four B fragments
//            of that product as four contiguous 1 KB runs: run (k % 64) / 16, then [q % 32][k % 16].
//            fp16 rather than fp32: the bias is half of what the attention core pulls in from L2
//            per key tile, and that traffic is a sixth of its run time; fp16's 11 significant
//            bits put its rounding (2^-12 of a logit) below that of the bf16 probabilities (2^-9).
//            Entries whose key is >= N are zero; query rows >= N of the last block are unused.
__host__ __device__ inline int64_t tri_ldn(int64_t n) { return (n + 15) / 16 * 16; }
__host__ __device__ inline int tri_vt_pos(int k) { return (k & ~12) | ((k & 8) >> 1) | ((k & 4) << 1); }
__host__ __device__ inline int64_t tri_bias_qblocks(int64_t n) { return (n + 31) / 32; }
__host__ __device__ inline int64_t tri_bias_ktiles(int64_t n) { return (n + 63) / 64; }
__host__ __device__ inline int64_t tri_bias_elems(int64_t n, int64_t heads) {
  return heads * tri_bias_qblocks(n) * tri_bias_ktiles(n) * 2048;
}
__host__ __device__ inline int64_t tri_bias_offset(int64_t n, int h, int q, int k) {
  return ((((int64_t)h * tri_bias_qblocks(n) + (q >> 5)) * tri_bias_ktiles(n) + (k >> 6)) * 4 + ((k & 63) >> 4)) * 512 +
         (q & 31) * 16 + (k & 15);
}

struct TriAttnProjArgs {
  LnWidth lw;
  const void* pair = nullptr;  // [N][N][128]
  int io_f32 = 0, N = 0, transpose = 0, skip_ln = 0;
  const float *ln_w = nullptr, *ln_b = nullptr;
  const bf16_t* w_qkvg = nullptr;  // [4][128][128]: q, k, v chunks are used here (the gate chunk by attn_out)
  const bf16_t* w_bias = nullptr;  // [32][128], rows >= 4 zero
  int n_bias = 0;                  // 0 or 4
  float q_scale = 1.f, bias_scale = 1.f;
  bf16_t *q = nullptr, *k = nullptr, *vt = nullptr;
  uint16_t* bias = nullptr;  // fp16 bits, fragment order, tri_bias_elems(N, 4) elements
  int64_t ldn = 0;        // tri_ldn(N)
};
int launch_triattn_proj(const TriAttnProjArgs& a, hipStream_t stream);

struct TriAttnArgs {
  const bf16_t *q = nullptr, *k = nullptr, *vt = nullptr;
  const uint16_t* bias = nullptr;  // fp16 bits, fragment order (tri_bias_offset), or null
  const float* mask = nullptr;   // [N][N] 0/1 or null
  bf16_t* og = nullptr;          // [(b*N + s)][128] normalised attention output (the gate is applied by attn_out)
  int N = 0;
  int64_t ldn = 0;
};
int launch_triattn_flash(const TriAttnArgs& a, hipStream_t stream);

// --------------------------------------------------------------- check_f32.hip
struct CkGemmArgs {
  const float* A = nullptr;  // element (b, m, k) at A[b*sA + m*lda + k*ka]
  const float* B = nullptr;  // element (b, n, k) at B[b*sB + n*ldb + k*kb]
  float* C = nullptr;        // element (b, m, n) at C[b*sC + m*ldc + n]
  int M = 0, N = 0, K = 0, batch = 1;
  int64_t lda = 0, ka = 1, ldb = 0, kb = 1, ldc = 0, sA = 0, sB = 0, sC = 0;
  const float* bias = nullptr;  // y = sigmoid?((acc + bias) * alpha) * mul + add
  float alpha = 1.f;
  int sigmoid = 0;
  const float* mul = nullptr;   // [mul_rows][ld_mul], row m % mul_rows
  int64_t mul_rows = 0, ld_mul = 0;
  const float* add = nullptr;   // [b*s_add + m*ld_add + n]
  int64_t ld_add = 0, s_add = 0;
};
int launch_ck_gemm(const CkGemmArgs& g, hipStream_t s);

struct CkNormArgs {
  const float* x = nullptr;
  float* y = nullptr;
  int64_t rows = 0;
  int C = 0;
  const float *weight = nullptr, *bias = nullptr, *scale = nullptr, *shift = nullptr;
  int64_t cond_rows = 0, ld_cond = 0;
};
int launch_ck_norm(const CkNormArgs& a, hipStream_t s);

enum { CK_TRIMUL_SPLIT = 0, CK_CHAN_TO_PIX = 1, CK_TRANSPOSE_PIX = 2, CK_SWIGLU = 3, CK_BINARY = 4 };
int launch_ck_elementwise(int op, const float* x0, const float* x1, const float* x2, float* y0, float* y1,
                          int64_t n0, int64_t n1, int flag, hipStream_t s);

struct CkAttnArgs {
  const float *q = nullptr, *k = nullptr, *v = nullptr;  // base + batch*sb + pos*ss + head*d
  float* out = nullptr;
  int64_t q_sb = 0, q_ss = 0, k_sb = 0, k_ss = 0, v_sb = 0, v_ss = 0, o_sb = 0, o_ss = 0;
  int B = 0, H = 0, Sq = 0, Sk = 0, d = 0;
  const float* bias = nullptr;  // bias[bb*bias_sb + h*bias_sh + q*bias_sq + k*bias_sk]
  int64_t bias_sb = 0, bias_sh = 0, bias_sq = 0, bias_sk = 1;
  int bias_mod = 0;             // bb = b % bias_mod when > 0 (also indexes qpad / kpad)
  const float* key_mask = nullptr;  // [.][Sk], batch stride km_sb: 0 -> logit replaced by -1e9
  int64_t km_sb = 0;
  const float *qpad = nullptr, *kpad = nullptr;  // [.][Sq], [.][Sk]: +1e9 where both are 0
};
int launch_ck_attention(const CkAttnArgs& a, hipStream_t s);
