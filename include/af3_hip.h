/* C ABI of libaf3hip.so: the AlphaFold3 Pairformer / diffusion-transformer hot
 * path of hasaki321/Distributed-xfold as hand-written gfx950 (MI355X) kernels.
 *
 * Each entry point stands where one of the reference's fused CPU operators
 * (namespace `_alpha_attention`, src/distributed_xfold/xsmm_kernels/csrc/
 * Alpha_Attention.cpp:181-222) or one of the eager PyTorch steps wrapped around
 * them stands; the reference interface it replaces is cited on each.
 *
 * Conventions
 *  - All pointers are DEVICE pointers, 16-byte aligned, dense row-major unless a
 *    stride argument says otherwise.  Nothing here allocates, frees or
 *    synchronises: work is enqueued on `stream` and the caller owns every
 *    buffer, including the scratch `workspace` whose size the matching
 *    *_workspace_bytes function returns.
 *  - Activations of the residual stream are bf16 (AF3_BF16) or fp32 (AF3_F32);
 *    matrix operands are always rounded to bf16 for the MFMA units and
 *    accumulated in fp32.  Weights are bf16 in the packed layouts described per
 *    function (the host packs them once, as the reference's load_xsmm_params
 *    does); LayerNorm scales/offsets and biases are fp32.
 *  - Return value: AF3_OK (0) or a negative AF3_ERR_* code; af3_error_string
 *    names it.  A non-zero return means nothing was enqueued by the failing
 *    step.
 */
#ifndef AF3_HIP_H_
#define AF3_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AF3_OK 0
#define AF3_ERR_BAD_ARG (-1)
#define AF3_ERR_WORKSPACE (-2)
#define AF3_ERR_LAUNCH (-3)
#define AF3_ERR_UNSUPPORTED (-4)
#define AF3_ERR_TOO_LARGE (-5)

#define AF3_BF16 0
#define AF3_F32 1

typedef void* af3_stream_t; /* a hipStream_t */

/* Version of this interface; af3_abi_version() returns the value the library
 * was built with.  It changes whenever the meaning or layout of an argument of
 * an existing entry point changes, so a caller that packed operands for another
 * version can tell.  2: af3_grid_attention_core_forward takes no gate and
 * leaves the normalised, ungated output; its pair bias is fp16 in fragment
 * order and vt has its quads swapped (version 1 took a bf16 bias and a gate). */
#define AF3_ABI_VERSION 2
int af3_abi_version(void);
const char* af3_error_string(int code);

/* ---------------------------------------------------------------------------
 * Triangle multiplication.  Replaces
 *   torch.ops._alpha_attention.traingle_multiplication_forward
 *   (csrc/Alpha_Attention.cpp:148-169 schema :206-210; bodies
 *   csrc/triangle_multiplication{,_bf16}.h) together with the residual add of
 *   nn/d_pairformer.py:122-123.
 * act [N,N,128]; mask [N,N] fp32 0/1 or NULL; equation_flag 0 = outgoing
 * "ikc,jkc->ijc", 1 = incoming "kjc,kic->ijc" (prototypes/
 * TriangleMultiplication.py:34-38).  out [N,N,128] in io_dtype; with
 * residual != 0, out = act + update and out may alias act.
 * Packed weights:
 *   w_proj_gate [4][128][128]: chunk 0/1 = operand a, channels 0-63 / 64-127,
 *     chunk 2/3 = operand b; inside a chunk rows 0-63 are `projection` rows and
 *     rows 64-127 the matching `gate` rows.  Operand a of channel c is row 2c of
 *     the nn.Linear weight, operand b row 2c+1 (d_triangle_multiplication.py:
 *     162-165, de-interleave :128-129).
 *   w_gating_linear, w_output_projection [128][128] as stored by nn.Linear.
 */
size_t af3_triangle_multiplication_workspace_bytes(int64_t n_token);
int af3_triangle_multiplication_forward(
    const void* act, int io_dtype, const float* mask, int equation_flag,
    const float* left_norm_input_weight, const float* left_norm_input_bias,
    const uint16_t* w_proj_gate,
    const float* center_norm_weight, const float* center_norm_bias,
    const uint16_t* w_output_projection, const uint16_t* w_gating_linear,
    void* out, int residual, int64_t n_token,
    void* workspace, size_t workspace_bytes, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Triangle (grid) self-attention.  Replaces
 *   torch.ops._alpha_attention.grid_self_attn_forward
 *   (csrc/Alpha_Attention.cpp:50-70, schema :182-185; bodies
 *   csrc/grid_self_attention{,_bf16}.h) AND the eager steps
 *   DistributeGridSelfAttention.xsmm_forward wraps around it
 *   (nn/d_attention.py:58-85): LayerNorm, the 128->H pair-bias projection, the
 *   key-mask bias, the transpose for the ending-node operator and its inverse,
 *   plus the residual add of nn/d_pairformer.py:132,144.
 * pair [N,N,128]; mask [N,N] fp32 0/1 indexed (row of the possibly transposed
 * tensor, key) exactly as d_attention.py:63 uses it; masked keys are replaced by
 * -1e9.  act_norm_* NULL means `pair` is already normalised (operator-level
 * use).  Pair bias: either w_pair_bias ([roundup(H,32)][128], zero padded;
 * projected from LayerNorm(pair)) or a precomputed nonbatched_bias [H,N,N]
 * fp32, or neither.
 * Packed weights: w_qkvg [4][128][128] = q, k, v, gating_query as stored by
 * nn.Linear ([out, in]; equal to the reference's query_w[C,H,d] transposed and
 * flattened); w_output [128][128] likewise.  q is scaled by head_dim^-1/2.
 */
size_t af3_grid_self_attn_workspace_bytes(int64_t n_token, int num_head);
int af3_grid_self_attn_forward(
    const void* pair, int io_dtype, const float* mask, int transpose,
    const float* act_norm_weight, const float* act_norm_bias,
    const uint16_t* w_pair_bias, const float* nonbatched_bias,
    const uint16_t* w_qkvg, const uint16_t* w_output, int num_head,
    void* out, int residual, int64_t n_token,
    void* workspace, size_t workspace_bytes, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Transition (SwiGLU) on 128-channel activations, one fused kernel.  Replaces
 *   torch.ops._alpha_attention.transition_forward
 *   (csrc/Alpha_Attention.cpp:116-125, schema :187-189; body csrc/transition.h)
 *   and DistributeTransition.forward (nn/d_primitives.py:31-35), plus the
 *   residual add of nn/d_pairformer.py:146.
 * act [rows,128]; w1 [hidden/64][128][128]: slab s holds transition1 rows
 * 64s..64s+63 (the silu half) followed by rows hidden+64s..hidden+64s+63 (the
 * linear half); w2 [128][hidden] as stored by nn.Linear.  hidden = factor*128.
 */
int af3_transition_forward(
    const void* act, int io_dtype,
    const float* layernorm_weight, const float* layernorm_bias,
    const uint16_t* w1_packed, const uint16_t* w2, int hidden,
    void* out, int residual, int64_t rows, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * The three pair operators above on FEWER than 128 pair channels: the Pairformer
 * blocks of the template embedding run on 64 (nn/d_template.py:198-201:
 * PairformerBlock(c_pair=64, num_intermediate_factor=2, with_single=False)),
 * through the same reference operators as the 128-channel trunk.  The caller
 * zero-pads the channel axis: the tensor is [N,N,128] with channels
 * valid_channels..127 zero, LayerNorm weights and biases are zero there, and
 * every weight matrix has zero rows / columns for the padded channels (for the
 * attention each head's valid_channels/num_head dimensions sit at the front of
 * a 32-wide slot).  The kernels are the 128-channel ones; valid_channels only
 * tells the LayerNorms how many channels their statistics cover and the
 * attention what head dimension scales its logits.  The padded output channels
 * come out zero, so a residual stream stays padded.  Same arguments, workspace
 * sizes and error codes as the un-suffixed entry points otherwise; with
 * valid_channels = 128 the results are the same bits.
 */
int af3_triangle_multiplication_forward_padded(
    const void* act, int io_dtype, const float* mask, int equation_flag,
    const float* left_norm_input_weight, const float* left_norm_input_bias,
    const uint16_t* w_proj_gate,
    const float* center_norm_weight, const float* center_norm_bias,
    const uint16_t* w_output_projection, const uint16_t* w_gating_linear,
    void* out, int residual, int64_t n_token, int valid_channels,
    void* workspace, size_t workspace_bytes, af3_stream_t stream);
int af3_grid_self_attn_forward_padded(
    const void* pair, int io_dtype, const float* mask, int transpose,
    const float* act_norm_weight, const float* act_norm_bias,
    const uint16_t* w_pair_bias, const float* nonbatched_bias,
    const uint16_t* w_qkvg, const uint16_t* w_output, int num_head,
    void* out, int residual, int64_t n_token, int valid_channels,
    void* workspace, size_t workspace_bytes, af3_stream_t stream);
int af3_transition_forward_padded(
    const void* act, int io_dtype,
    const float* layernorm_weight, const float* layernorm_bias,
    const uint16_t* w1_packed, const uint16_t* w2, int hidden,
    void* out, int residual, int64_t rows, int valid_channels, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Pair-biased gated self-attention without output projection.  Replaces
 *   torch.ops._alpha_attention.batch_diffusion_self_attention_forward
 *   (csrc/Alpha_Attention.cpp:72-92, schema :191-194; bodies
 *   csrc/batch_diffusion_self_attention{,_bf16}.h), used for the Pairformer
 *   single attention and the diffusion transformer
 *   (nn/d_diffusion_transformer.py:197-218).
 * q_data [B,S,C] bf16, already (adaptive-)LayerNorm-ed; key_mask fp32 0/1
 * (masked keys replaced by -1e9) or NULL: [S] shared by the batch
 * (mask_batches = 1) or [B,S], one per batch entry as the reference operator's
 * bias [B,1,1,S] is (mask_batches = B); nonbatched_bias [H,S,S] fp32 shared by
 * the batch, or NULL; with bias_quad_major = 1 (S a multiple of 4) it is given
 * as [H,S/4,S,4], element (h, q, k) at ((h * S/4 + k/4) * S + q) * 4 + k%4: the
 * kernel's lanes hold consecutive queries, so this order makes its bias loads
 * contiguous (worth it for a bias that is computed once and used many times).
 * w_qkvg [4C][C] bf16 = q, k, v, gating_query rows as
 * stored by nn.Linear; query_b [C] fp32 or NULL.  head_dim = C/H in {16, 24, 32, 48}.
 * out [B,S,H,head_dim] (= [B,S,C]) in out_dtype: sigmoid(gate) * softmax(..) v.
 */
size_t af3_batch_diffusion_self_attention_workspace_bytes(int64_t batch, int64_t seq, int channels);
int af3_batch_diffusion_self_attention_forward(
    const uint16_t* q_data, const float* key_mask, int64_t mask_batches, const float* nonbatched_bias,
    int bias_quad_major, const uint16_t* w_qkvg, const float* query_b, int num_head,
    void* out, int out_dtype, int64_t batch, int64_t seq, int channels,
    void* workspace, size_t workspace_bytes, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * The same operator for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops (the diffusion sampler evaluates this attention
 * 24 x 200 times per batch), harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  Arguments and result are exactly those of
 * af3_batch_diffusion_self_attention_forward minus the workspace: the q / k /
 * v / gate scratch [batch * seq][4 * channels] bf16 lives in a device array the
 * library owns (AF3_STATIC_SCRATCH_BYTES on every GPU the library is used on,
 * held until the process ends).  The call allocates and frees nothing.
 * Limit: batch * seq * channels * 8 bytes <= AF3_STATIC_SCRATCH_BYTES (e.g. 5
 * samples x 768 tokens x 768 channels, or 1536 tokens x 384 channels);
 * beyond it the call returns AF3_ERR_TOO_LARGE and enqueues nothing.
 * All calls on one GPU share that GPU's array: calls that may overlap in time
 * on one GPU (different streams, different threads) race on it - serialise
 * them, or use the workspace-taking entry point.  The array keeps the previous
 * call's contents; nothing in it needs clearing (every element a call reads
 * was written by that call first).  The first call on a device looks the
 * array's device address up (no allocation); make that call outside of graph
 * capture.
 */
#define AF3_STATIC_SCRATCH_BYTES ((size_t)32 << 20)
int af3_batch_diffusion_self_attention_forward_static(
    const uint16_t* q_data, const float* key_mask, int64_t mask_batches, const float* nonbatched_bias,
    int bias_quad_major, const uint16_t* w_qkvg, const float* query_b, int num_head,
    void* out, int out_dtype, int64_t batch, int64_t seq, int channels, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Windowed (atom) cross-attention without output projection.  Replaces
 *   torch.ops._alpha_attention.batch_diffusion_cross_attention_forward
 *   (csrc/Alpha_Attention.cpp:127-146, schema :201-204; bodies
 *   csrc/batch_diffusion_cross_attention{,_bf16}.h) and the bias construction
 *   of DistrubuteCrossAttention.xsmm_forward (nn/d_diffusion_transformer.py:
 *   400-417).
 * q_data [B,Sq,C], m_data [B,Sk,C] bf16 (already adaptive-LayerNorm-ed), B =
 * samples * subsets.  Bias = pair_logits[b % bias_batches][H][Sq][Sk] (fp32 or
 * NULL) + 1e9 where mask_q[b % bias_batches][q] == 0 and
 * mask_k[b % bias_batches][k] == 0 (masks fp32 0/1 or both NULL).  A fully
 * batched bias [B,H,Sq,Sk], as the reference operator takes, is the case
 * bias_batches == B with NULL masks.
 * w_qg [2C][C] = q_projection, gating_query; w_kv [2C][C] = k_projection,
 * v_projection (nn.Linear layout); query_b [C] fp32.
 */
size_t af3_batch_diffusion_cross_attention_workspace_bytes(int64_t batch, int64_t sq, int64_t sk, int channels);
int af3_batch_diffusion_cross_attention_forward(
    const uint16_t* q_data, const uint16_t* m_data,
    const float* pair_logits, const float* mask_q, const float* mask_k, int64_t bias_batches,
    const uint16_t* w_qg, const uint16_t* w_kv, const float* query_b, int num_head,
    void* out, int out_dtype, int64_t batch, int64_t sq, int64_t sk, int channels,
    void* workspace, size_t workspace_bytes, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * The same cross-attention with the key windows gathered inside the kernel.
 * Replaces the sequence `atom_layout.convert(queries_to_keys, queries_act)`
 * (nn/d_diffusion_transformer.py:519-523) -> adaptive LayerNorm of the keys ->
 * batch_diffusion_cross_attention_forward for the case the reference always
 * has in the atom transformers: every key of a window is one of the query
 * atoms (or a masked slot).  K and V are then projected once per atom instead
 * of once per (window, key), a quarter of the rows at 128 keys per 32 queries.
 * q_data [B,Sq,C] as above with B = samples * bias_batches; atom_data
 * [samples, n_atoms, C] bf16, the adaptive-LayerNorm-ed key input of every atom;
 * key_rows [bias_batches, Sk] int32: row of atom_data that key k of window b is,
 * or negative for a masked slot (K = V = 0, as the reference's zeroed gather
 * gives).  Everything else as in af3_batch_diffusion_cross_attention_forward.
 */
size_t af3_gathered_cross_attention_workspace_bytes(int64_t batch, int64_t sq, int64_t samples, int64_t n_atoms,
                                                    int channels);
int af3_gathered_cross_attention_forward(
    const uint16_t* q_data, const uint16_t* atom_data, const int32_t* key_rows,
    const float* pair_logits, const float* mask_q, const float* mask_k, int64_t bias_batches,
    const uint16_t* w_qg, const uint16_t* w_kv, const float* query_b, int num_head,
    void* out, int out_dtype, int64_t batch, int64_t sq, int64_t sk, int64_t samples, int64_t n_atoms, int channels,
    void* workspace, size_t workspace_bytes, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Batched product c[i] = a[i] b[i]^T, a [batch][m][k], b [batch][n][k],
 * c [batch][m][n], all bf16 and contiguous, k a multiple of 8.  The triangle
 * contraction `cik,cjk->cij` of nn/d_triangle_multiplication.py:118-124 for a
 * pair width other than 128 (the 64-channel Pairformer blocks of the template
 * embedding, nn/d_template.py:198-201); the 128-channel path has its own kernel
 * inside af3_triangle_multiplication_forward.
 */
int af3_batched_nt_product_forward(
    const uint16_t* a, const uint16_t* b, uint16_t* c, int64_t batch, int64_t m, int64_t n, int64_t k,
    af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * out[c][r] = in[r][c] for a contiguous bf16 matrix [rows][cols], rows and cols
 * multiples of 8.  The MSA operators sum over MSA rows (outer-product mean,
 * nn/d_primitives.py:63) or tokens (pair-weighted averaging, nn/d_attention.py:
 * 137), which their activations [rows, N, c] carry as outer indices; the dense
 * kernels want the summation index innermost in both operands.
 */
int af3_transpose_bf16_forward(const uint16_t* in, uint16_t* out, int64_t rows, int64_t cols, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Aggregation of per-atom activations to tokens, the tail of the atom
 * cross-attention encoder (nn/d_atom_cross_attention.py:322-331: conversion of
 * the projected query activations to the token-atom layout, ReLU, masked mean
 * over the atom slots of a token):
 *   out[b][t][c] = (sum over slots a with idx[t][a] >= 0 of
 *                   max(src[b][idx[t][a]][c], 0)) / count[t]
 * src [batch][n_src][channels] bf16, idx [n_out][slots] int32 (row of src, or
 * negative for an absent atom; every index < n_src), count [n_out] fp32 (the
 * divisor, > 0), out [batch][n_out][channels] fp32.  slots <= 32, channels a
 * multiple of 8.  The sum is taken in slot order in fp32.
 */
int af3_gathered_relu_mean_forward(const uint16_t* src, const int32_t* idx, const float* count, float* out,
                                   int64_t batch, int64_t n_src, int64_t n_out, int slots, int channels,
                                   af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Embedding of the noisy atom positions, the head of the atom cross-attention
 * encoder (nn/d_atom_cross_attention.py:195-207: conversion of the positions to
 * the query layout, the 3 -> channels projection, query mask, + conditioning):
 *   out[b][q][c] = cond[q][c] + sum_k positions[b][rows[q]][k] * weight[c][k]
 * positions [batch][n_slots][3] fp32, rows [n_queries] int32 (slot of the
 * query's atom, or negative for a query without atom / masked query: the
 * position term is then zero), weight [channels][3] fp32, cond
 * [n_queries][channels] fp32, out [batch][n_queries][channels] in out_dtype.
 */
int af3_atom_position_features_forward(const float* positions, const int32_t* rows, const float* weight,
                                       const float* cond, void* out, int out_dtype, int64_t batch, int64_t n_slots,
                                       int64_t n_queries, int channels, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Broadcast of the token activations to the atoms at the head of the atom
 * cross-attention decoder (nn/d_atom_cross_attention.py:371-392: the projected
 * token rows converted to the query layout, + the encoder's skip connection,
 * query mask):
 *   out[b][q][c] = (rows[q] >= 0 ? src[b][rows[q]][c] : 0) + add[b][q][c]
 * src [batch][n_src][channels] bf16 (one row per token), rows [n_queries] int32
 * (token of the query's atom, negative for none), add and out
 * [batch][n_queries][channels] bf16 (the skip connection is zero where the
 * query mask is, so no further masking is needed).  The sum is taken in fp32
 * and rounded once.
 */
int af3_gather_rows_add_forward(const uint16_t* src, const int32_t* rows, const uint16_t* add, uint16_t* out,
                                int64_t batch, int64_t n_src, int64_t n_queries, int channels, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * The tail of the atom cross-attention decoder
 * (nn/d_atom_cross_attention.py:404-414: LayerNorm of the query activations,
 * projection to a position update, conversion to the token-atom layout):
 *   out[b][t][k] = rows[t] >= 0 ? sum_c y[c] * weight[k][c] : 0,   k = 0..2,
 *   y = LayerNorm(x[b][rows[t]]) * ln_weight, rounded to bf16 as the eager
 *   LayerNorm output is.
 * x [batch][n_src][128] bf16, rows [n_out] int32 (query of the atom slot, or
 * negative for an absent atom), ln_weight [128] fp32, weight [3][128] fp32,
 * out [batch][n_out][3] fp32.  channels must be 128.
 */
int af3_position_update_forward(const uint16_t* x, const int32_t* rows, const float* ln_weight, const float* weight,
                                float* out, int64_t batch, int64_t n_src, int64_t n_out, int channels,
                                af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Pair-logit projection: out[h][i][j] = (LayerNorm(pair)[i][j] . w[h]).
 * Replaces the eager `single_pair_logits_projection(single_pair_logits_norm(
 * pair)).permute(2,0,1)` of nn/d_pairformer.py:160-162 and the
 * `pair_logits_projection` + rearrange of nn/d_diffusion_transformer.py:299-305.
 * pair [N,N,128]; norm_bias may be NULL; w [roundup(n_out,32)][128] zero padded.
 * out [n_out][N][N] fp32.
 */
int af3_pair_logits_forward(
    const void* pair, int io_dtype, const float* norm_weight, const float* norm_bias,
    const uint16_t* w, int n_out, float* out, int64_t n_token, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Row LayerNorm / adaptive LayerNorm -> bf16.  Replaces fastnn.LayerNorm on
 * the single / diffusion / atom activations and AdaptiveLayerNorm.forward
 * (nn/d_diffusion_transformer.py:61-74):
 *   y = LN(x) [* weight + bias];  if scale: y = sigmoid(scale[r]) * y + shift[r],
 *   r = row % cond_rows (the conditioning is shared by the sample batch).
 * x [rows,C] in x_dtype, y [rows,C] bf16, scale/shift fp32 with `cond_rows`
 * rows of stride `cond_ld` elements (so both can live in one [cond_rows, 2C]
 * projection output).
 */
int af3_layer_norm_forward(
    const void* x, int x_dtype, uint16_t* y, int64_t rows, int channels,
    const float* weight, const float* bias,
    const float* scale, const float* shift, int64_t cond_rows, int64_t cond_ld,
    af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Dense projection y = epilogue(x W^T) on bf16 MFMA.  Replaces the eager
 * nn.Linear / fastnn.gated_linear_unit / AdaLNZero steps around the fused
 * operators (nn/d_diffusion_transformer.py:99-118, 142-145; nn/d_primitives.py:
 * 33-34).  x [M,K] bf16, w [N,K] bf16 (nn.Linear layout).
 *  mode AF3_LINEAR_PLAIN : y = (x W^T + bias) * alpha, optional sigmoid; y [M,N]
 *  mode AF3_LINEAR_SWIGLU: y = silu(a) * b, y [M,N/2] bf16; w rows packed in
 *        blocks of 64: 32 rows of the silu half, then the 32 matching rows of
 *        the linear half
 *  mode AF3_LINEAR_GATE_RES: y = residual + gate[m % gate_rows] * (x W^T + bias)
 *        (gate fp32 [gate_rows,N] or NULL, its rows gate_ld floats apart
 *        (0 = N: contiguous), so that one slice of a wider projection can be
 *        used in place; residual in res_dtype or NULL)
 *  mode AF3_LINEAR_REGROUP32: PLAIN, with element (m, n) stored at
 *        y[(m/32, n/32)][(m%32, n%32)], y [(M/32)*(N/32), 1024] (M, N multiples
 *        of 32).  With x = [(token b, channel c), msa row] and w = [(token d,
 *        channel e), msa row] this is the outer-product sum of
 *        nn/d_primitives.py:63-64, laid out for the contraction with output_w.
 *  mode AF3_LINEAR_ROWGATE_RES: GATE_RES with one factor per row,
 *        y = residual + gate[m % gate_rows] * (x W^T + bias), gate fp32 [gate_rows]
 *        (the division by the coverage count of nn/d_primitives.py:69-70)
 */
#define AF3_LINEAR_PLAIN 0
#define AF3_LINEAR_SWIGLU 2
#define AF3_LINEAR_GATE_RES 3
#define AF3_LINEAR_REGROUP32 4
#define AF3_LINEAR_ROWGATE_RES 5
int af3_linear_forward(
    const uint16_t* x, const uint16_t* w, const float* bias,
    void* y, int y_dtype, int64_t m, int n, int k,
    int mode, float alpha, int sigmoid,
    const float* gate, int64_t gate_rows, int64_t gate_ld,
    const void* residual, int res_dtype, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Softmax of the MSA pair-weighted averaging (nn/d_attention.py:131-133): the
 * pair logits [heads * N][N] fp32 plus the additive key mask 1e9 (mask - 1)
 * (key_mask [N] fp32 0/1, or NULL), normalised over the keys, as bf16 with rows
 * out_ld >= cols elements apart and the tail columns zero (the layout the
 * averaging product reads).
 */
int af3_masked_softmax_rows_forward(const float* logits, const float* key_mask, uint16_t* out, int64_t rows,
                                    int64_t cols, int64_t out_ld, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * The narrow fp32 layers of the atom conditioning (nn/d_atom_cross_attention.py:
 * 139-140, 161-162, 182-184: single-to-pair conditioning 128 -> 16 and the three
 * 16 -> 16 layers of the pair MLP; :407-411: the 128 -> 3 position update):
 *   y[r] = (residual ? residual[r] : 0) + W f(x[r]),  f = relu (relu_input) or identity,
 * x [rows,k] fp32, W [n_out,k] fp32 (nn.Linear layout), n_out 16 or 3, k a multiple
 * of 4 up to 128, y and residual [rows,n_out] fp32.  Plain fp32 FMAs.
 */
int af3_narrow_linear_f32_forward(const float* x, const float* w, const float* residual, float* y, int64_t rows,
                                  int k, int n_out, int relu_input, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Pair conditioning of the windowed atom attention
 * (nn/d_atom_cross_attention.py:231-311: row + column conditioning, the trunk pair
 * conditioning of the two atoms' tokens, offset / distance / validity embeddings of
 * atoms in one reference frame, then the three-layer MLP with its residual), one
 * pass per (subset, query, key), 16 channels, fp32:
 *   a   = row[s,q] + col[s,k] + [both atoms exist] token_pair[query_token[s,q], key_token[s,k]]
 *         + valid (W_off d + W_dist / (1 + |d|^2) + w_valid),  d = query_pos[s,q] - key_pos[s,k],
 *         valid = query_uid[s,q] == key_uid[s,k]
 *   out = a + W3 relu(W2 relu(W1 relu(a)))
 * row [subsets,queries,16], col [subsets,keys,16], token_pair [n_token,n_token,16] (or
 * null: no such term), query_token / key_token int32 (negative: no atom in the slot),
 * positions [.,3], uids int32, weights in nn.Linear layout ([16,3], [16,1], [16,1],
 * [16,16] x 3, no bias), out [subsets,queries,keys,16].
 */
int af3_atom_pair_cond_forward(const float* row, const float* col, const float* token_pair, const int32_t* query_token,
                               const int32_t* key_token, int64_t n_token, const float* query_pos, const float* key_pos,
                               const int32_t* query_uid, const int32_t* key_uid, const float* w_offsets,
                               const float* w_distances, const float* w_valid, const float* w_mlp1, const float* w_mlp2,
                               const float* w_mlp3, float* out, int64_t subsets, int64_t queries, int64_t keys,
                               af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Pair logits of the windowed atom transformer for all its blocks
 * (nn/d_diffusion_transformer.py:510-520: pair_input_layer_norm, then
 * pair_logits_projection, then the split into blocks and heads), one pass, fp32:
 *   pair_cond [subsets,queries,keys,16] fp32, ln_w [16] fp32 (the norm has no bias),
 *   w [num_blocks*num_head,16] fp32 (nn.Linear layout, no bias; at most 32 rows),
 *   out [num_blocks,subsets,num_head,queries,keys] fp32.
 */
int af3_atom_pair_logits_forward(const float* pair_cond, const float* ln_w, const float* w, float* out, int64_t subsets,
                                 int64_t queries, int64_t keys, int num_blocks, int num_head, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Pair conditioning of the diffusion head, first layer
 * (nn/d_diffusion_head.py:104-116: features_2d = [pair | relative encoding],
 * pair_cond = pair_cond_initial_projection(pair_cond_initial_norm(features_2d))),
 * in one pass and without the concatenated [n,n,267] tensor.  The relative
 * encoding of the token pair (i, j) is one-hot: clipped residue offset inside a
 * chain (2 r + 2 classes, the last for different chains), clipped token offset
 * inside a residue (2 r + 2), same entity (1), clipped chain-copy offset inside an
 * entity (2 c + 2); r = max_relative_idx, c = max_relative_chain, n_rel = 4 r + 2 c + 7
 * channels after the 128 of `pair`.
 *   pair      [n,n,128] fp32 or bf16 (pair_dtype), multiplied by in_scale first
 *   asym_id .. sym_id   [n] int32 token features
 *   ln_w      [128] fp32: LayerNorm weights of the pair channels (the norm has no bias)
 *   w_pair    [128,128] bf16: projection weights of the pair channels, W[:, :128]
 *   g_hot     [n_rel,128] fp32: g_hot[h][o] = ln_w[128 + h] * W[o][128 + h]
 *   g_sum     [128] fp32: sum over h of g_hot[h][o]
 *   out       [n,n,128] fp32
 */
int af3_pair_cond_init_forward(const void* pair, int pair_dtype, float in_scale, const int32_t* asym_id,
                               const int32_t* residue_index, const int32_t* token_index, const int32_t* entity_id,
                               const int32_t* sym_id, int max_relative_idx, int max_relative_chain, const float* ln_w,
                               const uint16_t* w_pair, const float* g_hot, const float* g_sum, float* out, int64_t n,
                               af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * Diagnostic, no counterpart in the reference.  The dense kernels fetch a
 * column bias in groups (eight entries on the 128x128 tile, four per lane on the
 * 256x256 tile, the last group pulled back to end at column n), and a segmented
 * epilogue (the q-k-v-gate projection of the attentions: segments of seg_len
 * columns, op of segment s in bits [4s, 4s+4) of seg_ops, 1 = biased and
 * scaled) only touches the entries of the segments that use the bias.
 * af3_linear_bias_span reports the half-open range [*first, *last) of entries
 * a product x[m,k] W[n,k]^T with a bias would read on the kernel that takes it
 * (seg_len = 0: one bias per column, as af3_linear_forward), computed by the
 * function the launch path itself checks the caller's extent with; no GPU is
 * needed.
 */
int af3_linear_bias_span(int64_t m, int n, int k, int seg_len, int seg_ops, int64_t* first, int64_t* last);

/* ---------------------------------------------------------------------------
 * Kernel-level entry points: the two MFMA-bound inner kernels on their own,
 * so that a caller (the benchmark's roofline leg, a profiler) can time exactly
 * one launch.  They are the inner stages of the operators above.
 *
 * af3_triangle_contraction_forward: t[c][i][j] = sum_k a[c][i][k] * b[c][j][k]
 *   for 128 channels, the contraction stage of the triangle multiplication
 *   (csrc/triangle_multiplication_bf16.h:257-401).  a, b, t are channel-major
 *   bf16 [128][n_token][ld] with ld = n_token rounded up to 8; columns
 *   n_token..ld-1 of a and b must be zero.
 * af3_grid_attention_core_forward: the flash attention stage of the triangle
 *   attention (csrc/grid_self_attention_bf16.h:226-481) on already projected
 *   operands, head-major, in base-2 form (4 heads of 32, ld = n_token rounded
 *   up to 16):
 *     q  bf16 [b][h][s][32] = query * log2(e)/sqrt(32);  k bf16 [b][h][s][32];
 *     vt bf16 [b][h][32][ld] = value transposed, key k of a row stored at column
 *       (k & ~12) | ((k & 8) >> 1) | ((k & 4) << 1) (inside every aligned group of 16 keys
 *       the two middle quads are swapped), columns of keys >= n_token zero;
 *     pair_bias fp16 = bias * log2(e) in MFMA-fragment order, or NULL: element (h, q, k) at
 *       ((((h*QB + q/32)*KT + k/64)*4 + (k%64)/16)*32 + q%32)*16 + k%16,
 *       QB = ceil(N/32), KT = ceil(N/64), 4*QB*KT*2048 elements, keys >= N zero
 *       (per head, 32-query block and 64-key tile: four contiguous 1 KB runs, each
 *       the B operand of one identity-matrix MFMA that adds the bias to the logits);
 *   key mask [N][N] fp32 0/1 or NULL;
 *   og [(b*N + s)][128] = softmax(q k^T + bias) v  (the output gate, sigmoid(LN(x) Wg^T), is
 *   applied by the operator's last kernel together with the output projection).
 */
int af3_triangle_contraction_forward(
    const uint16_t* a, const uint16_t* b, uint16_t* t, int64_t n_token, af3_stream_t stream);
int af3_grid_attention_core_forward(
    const uint16_t* q, const uint16_t* k, const uint16_t* vt,
    const uint16_t* pair_bias, const float* mask, uint16_t* og, int64_t n_token, af3_stream_t stream);

/* ---------------------------------------------------------------------------
 * fp32 check mode.  Plain fp32 kernels (fp32 storage, fp32 FMA arithmetic, no
 * MFMA, no fusion) from which the host composes every operator above a second
 * time; they share no code with the bf16 kernels.  They have no counterpart in
 * the reference's operator set: they exist so that the bf16 path can be checked
 * on the GPU, at sizes the CPU oracle cannot reach, against an independent
 * implementation that itself matches the oracle to 1e-4.
 *
 * af3_check_gemm_f32: C[b][m][n] = (sigmoid?)((sum_k A(b,m,k) B(b,n,k) + bias[n]) * alpha)
 *   * mul[m % mul_rows][n] + add(b,m,n), with A(b,m,k) = a[b*sa + m*lda + k*ka] and
 *   B(b,n,k) = b[b*sb + n*ldb + k*kb] (so either operand may be read transposed).
 * af3_check_layer_norm_f32: the fp32 twin of af3_layer_norm_forward.
 * af3_check_elementwise_f32: op 0 triangle-multiplication gating and a/b split
 *   (x0 proj [N*N,2c], x1 gate, x2 mask or NULL -> y0 a, y1 b channel-major
 *   [c][N][N], c = n1 or 128 if n1 is 0; flag 1 = incoming, stored transposed), op 1 channel-major
 *   [n1][N][N] -> [N][N][n1], op 2 out[j][i][:] = in[i][j][:] with n1 channels,
 *   op 3 SwiGLU y0[m][f] = silu(x0[m][f]) * x0[m][n1 + f] for n0 rows,
 *   op 4 y0 = x0 * x1 (flag 0) or x0 + x1 (flag 1) over n0 elements.
 * af3_check_attention_f32: softmax(q.k + bias, masks) v per (batch, head, query),
 *   operands addressed base + batch*sb + position*ss + head*head_dim, bias at
 *   bias[(b % bias_mod)*bias_sb + h*bias_sh + q*bias_sq + k*bias_sk]; key_mask /
 *   qpad / kpad as in the bf16 entry points.
 */
int af3_check_gemm_f32(
    const float* a, const float* b, float* c, int64_t m, int64_t n, int64_t k, int64_t batch,
    int64_t lda, int64_t ka, int64_t ldb, int64_t kb, int64_t ldc, int64_t sa, int64_t sb, int64_t sc,
    const float* bias, float alpha, int sigmoid, const float* mul, int64_t mul_rows, int64_t ld_mul,
    const float* add, int64_t ld_add, int64_t s_add, af3_stream_t stream);
int af3_check_layer_norm_f32(
    const float* x, float* y, int64_t rows, int channels, const float* weight, const float* bias,
    const float* scale, const float* shift, int64_t cond_rows, int64_t cond_ld, af3_stream_t stream);
int af3_check_elementwise_f32(
    int op, const float* x0, const float* x1, const float* x2, float* y0, float* y1,
    int64_t n0, int64_t n1, int flag, af3_stream_t stream);
int af3_check_attention_f32(
    const float* q, const float* k, const float* v, float* out,
    int64_t q_sb, int64_t q_ss, int64_t k_sb, int64_t k_ss, int64_t v_sb, int64_t v_ss, int64_t o_sb, int64_t o_ss,
    int64_t batch, int num_head, int64_t sq, int64_t sk, int head_dim,
    const float* bias, int64_t bias_sb, int64_t bias_sh, int64_t bias_sq, int64_t bias_sk, int64_t bias_mod,
    const float* key_mask, int64_t km_sb, const float* qpad, const float* kpad, af3_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* AF3_HIP_H_ */
