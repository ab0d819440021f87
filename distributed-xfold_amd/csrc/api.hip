// C ABI of libaf3hip.so (declared in include/af3_hip.h): argument checks,
// workspace carving and kernel sequencing.  No allocation, no synchronisation.
#include "../../include/af3_hip.h"
#include "kernels.h"
#include <mutex>

namespace {

constexpr int C_PAIR = 128;

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
inline int64_t pad8(int64_t n) { return (n + 7) / 8 * 8; }

// bump allocator over the caller's workspace
struct Carver {
  char* base;
  size_t size, used = 0;
  bool ok = true;
  Carver(void* p, size_t n) : base(static_cast<char*>(p)), size(n) {}
  template <typename T> T* take(size_t count) {
    const size_t bytes = align_up(count * sizeof(T), 256);
    if (!base || used + bytes > size) { ok = false; return nullptr; }
    T* r = reinterpret_cast<T*>(base + used);
    used += bytes;
    return r;
  }
};

inline bool bad_dtype(int d) { return d != AF3_BF16 && d != AF3_F32; }
inline bool misaligned(const void* p) { return ((uintptr_t)p & 15) != 0; }

}  // namespace

// ---------------------------------------------------------------------------
// Library-owned scratch of the allocation-free entry point.  The array lives in
// this code object's device data segment: every GPU the library runs on holds
// its own copy, at its own address, from the moment the code object is loaded
// there until the process ends.  In host code the NAME `scratch` is only a
// handle for hipGetSymbolAddress, never an address a kernel could use; the
// device address is looked up once per device and kept.
// ---------------------------------------------------------------------------
constexpr size_t STATIC_SCRATCH_BYTES = AF3_STATIC_SCRATCH_BYTES;   // 32 MiB
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

namespace {

constexpr int MAX_DEVICES = 64;
std::mutex scratch_lock;
void* scratch_dev_ptr[MAX_DEVICES] = {};

// Device address of `scratch` on the CURRENT device, or null on failure.
void* static_scratch_ptr() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> hold(scratch_lock);
  if (!scratch_dev_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
      (void)hipGetLastError();
      return nullptr;
    }
    scratch_dev_ptr[dev] = p;
  }
  return scratch_dev_ptr[dev];
}

}  // namespace

extern "C" {

int af3_abi_version(void) { return AF3_ABI_VERSION; }

const char* af3_error_string(int code) {
  switch (code) {
    case AF3_OK: return "ok";
    case AF3_ERR_BAD_ARG: return "bad argument (null/misaligned pointer, shape or dtype)";
    case AF3_ERR_WORKSPACE: return "workspace missing or too small";
    case AF3_ERR_LAUNCH: return "kernel launch failed";
    case AF3_ERR_UNSUPPORTED: return "unsupported shape (channels / head dimension)";
    case AF3_ERR_TOO_LARGE: return "problem exceeds the library-owned scratch of the allocation-free entry point";
    default: return "unknown error";
  }
}

// ------------------------------------------------------ triangle multiplication
// The N x N x N contraction of the triangle multiplication: the 256x256-tile
// kernel once a token count fills at least part of a second 128-row tile,
// the general 128x128-tile GEMM below that.
static int contraction(const GemmArgs& g, hipStream_t s) {
  if (g.M > 128 && contract_supported(g)) return launch_contract(g, s);
  return launch_gemm_nt(g, s);
}

size_t af3_triangle_multiplication_workspace_bytes(int64_t n) {
  if (n <= 0) return 0;
  return 3 * align_up((size_t)C_PAIR * n * pad8(n) * sizeof(bf16_t), 256);
}

static int triangle_multiplication_impl(
    const void* act, int io_dtype, const float* mask, int equation_flag,
    const float* ln_in_w, const float* ln_in_b, const uint16_t* w_proj_gate,
    const float* ln_c_w, const float* ln_c_b, const uint16_t* w_out, const uint16_t* w_gl,
    void* out, int residual, int64_t n, int valid_channels, void* workspace, size_t workspace_bytes,
    af3_stream_t stream) {
  if (!act || !out || !ln_in_w || !ln_in_b || !w_proj_gate || !ln_c_w || !ln_c_b || !w_out || !w_gl)
    return AF3_ERR_BAD_ARG;
  if (valid_channels < 8 || valid_channels > C_PAIR) return AF3_ERR_BAD_ARG;
  if (bad_dtype(io_dtype) || n <= 0 || n > 8192 || (equation_flag != 0 && equation_flag != 1)) return AF3_ERR_BAD_ARG;
  if (misaligned(act) || misaligned(out) || misaligned(mask)) return AF3_ERR_BAD_ARG;
  const int64_t np = pad8(n);
  Carver ws(workspace, workspace_bytes);
  bf16_t* a_buf = ws.take<bf16_t>((size_t)C_PAIR * n * np);
  bf16_t* b_buf = ws.take<bf16_t>((size_t)C_PAIR * n * np);
  bf16_t* t_buf = ws.take<bf16_t>((size_t)C_PAIR * n * np);
  if (!ws.ok) return AF3_ERR_WORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);

  TriMulArgs a;
  a.lw = ln_width(valid_channels);
  a.valid_c = valid_channels;
  a.pair = act; a.mask = mask; a.out = out;
  a.io_f32 = io_dtype == AF3_F32; a.N = (int)n; a.Np = (int)np;
  a.outgoing = equation_flag == 0; a.residual = residual != 0;
  a.ln_in_w = ln_in_w; a.ln_in_b = ln_in_b; a.ln_c_w = ln_c_w; a.ln_c_b = ln_c_b;
  a.w_pg = w_proj_gate; a.w_gl = w_gl; a.w_out = w_out;
  a.a_buf = a_buf; a.b_buf = b_buf; a.t_buf = t_buf;
  int rc = launch_trimul_prologue(a, s);
  if (rc) return rc;

  // outgoing: t[c][i][j] = sum_k a'[c][i][k] b'[c][j][k]
  // incoming: t[c][i][j] = sum_k b'[c][i][k] a'[c][j][k]  (a', b' stored transposed by the prologue)
  GemmArgs g;
  g.A = a.outgoing ? a_buf : b_buf;
  g.B = a.outgoing ? b_buf : a_buf;
  g.C = t_buf;
  // (the hidden layer has as many channels as the pair tensor: the padded ones are zero and are left out)
  g.M = g.N = (int)n; g.K = (int)np; g.batch = valid_channels;
  g.lda = g.ldb = g.ldc = np;
  g.sA = g.sB = g.sC = n * np;
  rc = contraction(g, s);
  if (rc) return rc;
  return launch_trimul_epilogue(a, s);
}

// ------------------------------------------------------------ triangle attention
size_t af3_grid_self_attn_workspace_bytes(int64_t n, int num_head) {
  if (n <= 0 || num_head <= 0) return 0;
  const size_t e = sizeof(bf16_t), ldn = (size_t)tri_ldn(n);
  // fast path: q, k planes, vt, og, fp16 bias
  const size_t fast = 2 * align_up((size_t)n * n * C_PAIR * e, 256) + align_up((size_t)n * C_PAIR * ldn * e, 256) +
                      align_up((size_t)n * n * C_PAIR * e, 256) +
                      align_up((size_t)tri_bias_elems(n, num_head) * sizeof(uint16_t), 256);
  // general path (external fp32 bias): qkv + og
  const size_t general = align_up((size_t)n * n * 3 * C_PAIR * e, 256) + align_up((size_t)n * n * C_PAIR * e, 256);
  return fast > general ? fast : general;
}

static int grid_self_attn_impl(
    const void* pair, int io_dtype, const float* mask, int transpose,
    const float* ln_w, const float* ln_b, const uint16_t* w_pair_bias, const float* nonbatched_bias,
    const uint16_t* w_qkvg, const uint16_t* w_output, int num_head,
    void* out, int residual, int64_t n, int valid_channels, void* workspace, size_t workspace_bytes,
    af3_stream_t stream) {
  if (!pair || !out || !w_qkvg || !w_output) return AF3_ERR_BAD_ARG;
  if (valid_channels < num_head || valid_channels > C_PAIR || (num_head > 0 && valid_channels % num_head))
    return AF3_ERR_BAD_ARG;
  if (bad_dtype(io_dtype) || n <= 0 || n > 8192 || num_head <= 0 || C_PAIR % num_head) return AF3_ERR_BAD_ARG;
  if ((ln_w == nullptr) != (ln_b == nullptr)) return AF3_ERR_BAD_ARG;
  if (w_pair_bias && nonbatched_bias) return AF3_ERR_BAD_ARG;
  if (misaligned(pair) || misaligned(out) || misaligned(mask) || misaligned(nonbatched_bias)) return AF3_ERR_BAD_ARG;
  const int d = C_PAIR / num_head;  // head dimension of the (padded) operands
  if (d != 32 || num_head != 4) return AF3_ERR_UNSUPPORTED;
  const float d_valid = (float)(valid_channels / num_head);  // what the logits are scaled by
  hipStream_t s = static_cast<hipStream_t>(stream);
  Carver ws(workspace, workspace_bytes);
  bf16_t* og = nullptr;
  int rc;
  if (nonbatched_bias == nullptr) {
    // Fast path: the pair bias (if any) is projected here, so everything the
    // attention core needs is produced in its preferred form: base-2 logits,
    // fp16 bias in fragment order, head-major planes, V transposed.
    const float LOG2E = 1.4426950408889634f;
    const int64_t ldn = tri_ldn(n);
    bf16_t* q = ws.take<bf16_t>((size_t)n * n * C_PAIR);
    bf16_t* k = ws.take<bf16_t>((size_t)n * n * C_PAIR);
    bf16_t* vt = ws.take<bf16_t>((size_t)n * C_PAIR * ldn);
    og = ws.take<bf16_t>((size_t)n * n * C_PAIR);
    uint16_t* bias = ws.take<uint16_t>((size_t)tri_bias_elems(n, num_head));
    if (!ws.ok) return AF3_ERR_WORKSPACE;
    TriAttnProjArgs p;
    p.lw = ln_width(valid_channels);
    p.pair = pair; p.io_f32 = io_dtype == AF3_F32; p.N = (int)n; p.transpose = transpose != 0;
    p.skip_ln = ln_w == nullptr; p.ln_w = ln_w; p.ln_b = ln_b;
    p.w_qkvg = w_qkvg; p.w_bias = w_pair_bias; p.n_bias = w_pair_bias ? num_head : 0;
    p.q_scale = LOG2E / sqrtf(d_valid); p.bias_scale = LOG2E;
    p.q = q; p.k = k; p.vt = vt; p.bias = bias; p.ldn = ldn;
    rc = launch_triattn_proj(p, s);
    if (rc) return rc;
    TriAttnArgs t;
    t.q = q; t.k = k; t.vt = vt; t.bias = w_pair_bias ? bias : nullptr;
    t.mask = mask; t.og = og; t.N = (int)n; t.ldn = ldn;
    rc = launch_triattn_flash(t, s);
    if (rc) return rc;
  } else {
    // General path: an external fp32 bias [H][N][N] (operator-level contract).
    bf16_t* qkv = ws.take<bf16_t>((size_t)n * n * 3 * C_PAIR);
    og = ws.take<bf16_t>((size_t)n * n * C_PAIR);
    if (!ws.ok) return AF3_ERR_WORKSPACE;
    AttnProjArgs p;
    p.lw = ln_width(valid_channels);
    p.pair = pair; p.io_f32 = io_dtype == AF3_F32; p.N = (int)n; p.transpose = transpose != 0;
    p.ln_w = ln_w; p.ln_b = ln_b; p.skip_ln = ln_w == nullptr;
    p.w_main = w_qkvg; p.n_chunks = 3;  // the gate chunk is applied by attn_out
    p.chunk_ops = SEG_BIAS_SCALE | (SEG_PLAIN << 4) | (SEG_PLAIN << 8);
    p.q_scale = 1.0f / sqrtf(d_valid);
    p.out_main = qkv; p.ld_main = 3 * C_PAIR;
    rc = launch_attn_proj(p, s);
    if (rc) return rc;
    FlashArgs f;
    f.q = qkv; f.k = qkv + C_PAIR; f.v = qkv + 2 * C_PAIR;
    f.q_ss = f.k_ss = f.v_ss = 3 * C_PAIR;
    f.q_sb = f.k_sb = f.v_sb = n * 3 * C_PAIR;
    f.out = og; f.out_f32 = 0; f.o_ss = C_PAIR; f.o_sb = n * C_PAIR;
    f.B = (int)n; f.H = num_head; f.Sq = f.Sk = (int)n; f.d = d;
    f.bias = nonbatched_bias; f.bias_sb = 0; f.bias_sh = n * n; f.bias_sq = n;
    f.key_mask = mask; f.km_sb = n;
    rc = launch_flash_attention(f, s);
    if (rc) return rc;
  }

  AttnOutArgs o;
  o.lw = ln_width(valid_channels);
  o.og = og; o.ld_og = C_PAIR; o.w_gate = w_qkvg + 3 * C_PAIR * C_PAIR; o.w_out = w_output; o.pair = pair; o.out = out;
  o.skip_ln = ln_w == nullptr; o.ln_w = ln_w; o.ln_b = ln_b;
  o.io_f32 = io_dtype == AF3_F32; o.N = (int)n; o.transpose = transpose != 0; o.residual = residual != 0;
  return launch_attn_out(o, s);
}

// -------------------------------------------------------------------- transition
static int transition_impl(
    const void* act, int io_dtype, const float* ln_w, const float* ln_b,
    const uint16_t* w1_packed, const uint16_t* w2, int hidden,
    void* out, int residual, int64_t rows, int valid_channels, af3_stream_t stream) {
  if (!act || !out || !ln_w || !ln_b || !w1_packed || !w2) return AF3_ERR_BAD_ARG;
  if (bad_dtype(io_dtype) || rows <= 0 || rows > 0x7fffffff || hidden <= 0 || (hidden & 63)) return AF3_ERR_BAD_ARG;
  if (valid_channels < 8 || valid_channels > C_PAIR) return AF3_ERR_BAD_ARG;
  TransitionArgs t;
  t.lw = ln_width(valid_channels);
  t.x = act; t.out = out; t.io_f32 = io_dtype == AF3_F32; t.N = (int)rows; t.hidden = hidden;
  t.residual = residual != 0; t.ln_w = ln_w; t.ln_b = ln_b; t.w1 = w1_packed; t.w2 = w2;
  return launch_transition(t, static_cast<hipStream_t>(stream));
}

// The public forms: all 128 channels real, or the tensor and every weight zero-padded to 128 channels
// with `valid_channels` of them real.
int af3_triangle_multiplication_forward(
    const void* act, int io_dtype, const float* mask, int equation_flag,
    const float* ln_in_w, const float* ln_in_b, const uint16_t* w_proj_gate,
    const float* ln_c_w, const float* ln_c_b, const uint16_t* w_out, const uint16_t* w_gl,
    void* out, int residual, int64_t n, void* workspace, size_t workspace_bytes, af3_stream_t stream) {
  return triangle_multiplication_impl(act, io_dtype, mask, equation_flag, ln_in_w, ln_in_b, w_proj_gate, ln_c_w, ln_c_b,
                                      w_out, w_gl, out, residual, n, C_PAIR, workspace, workspace_bytes, stream);
}
int af3_triangle_multiplication_forward_padded(
    const void* act, int io_dtype, const float* mask, int equation_flag,
    const float* ln_in_w, const float* ln_in_b, const uint16_t* w_proj_gate,
    const float* ln_c_w, const float* ln_c_b, const uint16_t* w_out, const uint16_t* w_gl,
    void* out, int residual, int64_t n, int valid_channels, void* workspace, size_t workspace_bytes,
    af3_stream_t stream) {
  return triangle_multiplication_impl(act, io_dtype, mask, equation_flag, ln_in_w, ln_in_b, w_proj_gate, ln_c_w, ln_c_b,
                                      w_out, w_gl, out, residual, n, valid_channels, workspace, workspace_bytes, stream);
}
int af3_grid_self_attn_forward(
    const void* pair, int io_dtype, const float* mask, int transpose,
    const float* ln_w, const float* ln_b, const uint16_t* w_pair_bias, const float* nonbatched_bias,
    const uint16_t* w_qkvg, const uint16_t* w_output, int num_head,
    void* out, int residual, int64_t n, void* workspace, size_t workspace_bytes, af3_stream_t stream) {
  return grid_self_attn_impl(pair, io_dtype, mask, transpose, ln_w, ln_b, w_pair_bias, nonbatched_bias, w_qkvg, w_output,
                             num_head, out, residual, n, C_PAIR, workspace, workspace_bytes, stream);
}
int af3_grid_self_attn_forward_padded(
    const void* pair, int io_dtype, const float* mask, int transpose,
    const float* ln_w, const float* ln_b, const uint16_t* w_pair_bias, const float* nonbatched_bias,
    const uint16_t* w_qkvg, const uint16_t* w_output, int num_head,
    void* out, int residual, int64_t n, int valid_channels, void* workspace, size_t workspace_bytes,
    af3_stream_t stream) {
  return grid_self_attn_impl(pair, io_dtype, mask, transpose, ln_w, ln_b, w_pair_bias, nonbatched_bias, w_qkvg, w_output,
                             num_head, out, residual, n, valid_channels, workspace, workspace_bytes, stream);
}
int af3_transition_forward(
    const void* act, int io_dtype, const float* ln_w, const float* ln_b,
    const uint16_t* w1_packed, const uint16_t* w2, int hidden,
    void* out, int residual, int64_t rows, af3_stream_t stream) {
  return transition_impl(act, io_dtype, ln_w, ln_b, w1_packed, w2, hidden, out, residual, rows, C_PAIR, stream);
}
int af3_transition_forward_padded(
    const void* act, int io_dtype, const float* ln_w, const float* ln_b,
    const uint16_t* w1_packed, const uint16_t* w2, int hidden,
    void* out, int residual, int64_t rows, int valid_channels, af3_stream_t stream) {
  return transition_impl(act, io_dtype, ln_w, ln_b, w1_packed, w2, hidden, out, residual, rows, valid_channels, stream);
}

// ------------------------------------------- pair-biased self-attention (single / diffusion)
size_t af3_batch_diffusion_self_attention_workspace_bytes(int64_t batch, int64_t seq, int channels) {
  if (batch <= 0 || seq <= 0 || channels <= 0) return 0;
  return align_up((size_t)batch * seq * 4 * channels * sizeof(bf16_t), 256);
}

// Argument checks and the two launches (q/k/v/gate product, flash kernel) shared by the
// workspace-taking entry point and the allocation-free one: `qkvg` is the scratch
// [batch * seq][4 * channels] bf16, wherever it lives.
static int self_attention_args_ok(
    const uint16_t* q_data, const float* key_mask, int64_t mask_batches, int bias_quad_major,
    const uint16_t* w_qkvg, void* out, int out_dtype, int num_head, int64_t batch, int64_t seq, int channels) {
  if (!q_data || !w_qkvg || !out) return AF3_ERR_BAD_ARG;
  if (bias_quad_major != 0 && (bias_quad_major != 1 || (seq & 3))) return AF3_ERR_BAD_ARG;
  if (bad_dtype(out_dtype) || batch <= 0 || seq <= 0 || channels <= 0 || (channels & 7) || num_head <= 0 ||
      channels % num_head)
    return AF3_ERR_BAD_ARG;
  if (batch * seq > 0x7fffffff) return AF3_ERR_BAD_ARG;
  if (key_mask && mask_batches != 1 && mask_batches != batch) return AF3_ERR_BAD_ARG;
  const int d = channels / num_head;
  if (d != 16 && d != 24 && d != 32 && d != 48) return AF3_ERR_UNSUPPORTED;
  return AF3_OK;
}

static int self_attention_run(
    const uint16_t* q_data, const float* key_mask, int64_t mask_batches, const float* nonbatched_bias,
    int bias_quad_major, const uint16_t* w_qkvg, const float* query_b, int num_head,
    void* out, int out_dtype, int64_t batch, int64_t seq, int channels, bf16_t* qkvg, hipStream_t s) {
  const int d = channels / num_head;
  GemmArgs g;
  g.A = q_data; g.B = w_qkvg; g.C = qkvg;
  g.M = (int)(batch * seq); g.N = 4 * channels; g.K = channels;
  g.lda = channels; g.ldb = channels; g.ldc = 4 * channels;
  g.epi = EPI_SEGMENTED; g.seg_len = channels;
  g.seg_ops = SEG_BIAS_SCALE | (SEG_PLAIN << 4) | (SEG_PLAIN << 8) | (SEG_SIGMOID << 12);
  g.alpha = 1.0f / sqrtf((float)d);
  g.bias = query_b; g.bias_len = channels;  // the query segment's columns only
  int rc = launch_gemm_nt(g, s);
  if (rc) return rc;

  FlashArgs f;
  f.q = qkvg; f.k = qkvg + channels; f.v = qkvg + 2 * channels; f.g = qkvg + 3 * channels;
  f.q_ss = f.k_ss = f.v_ss = f.g_ss = 4 * channels;
  f.q_sb = f.k_sb = f.v_sb = f.g_sb = seq * 4 * channels;
  f.out = out; f.out_f32 = out_dtype == AF3_F32; f.o_ss = channels; f.o_sb = seq * channels;
  f.B = (int)batch; f.H = num_head; f.Sq = f.Sk = (int)seq; f.d = d;
  f.bias = nonbatched_bias; f.bias_sb = 0; f.bias_sh = seq * seq; f.bias_sq = seq;
  if (bias_quad_major) { f.bias_sq = 4; f.bias_squad = seq * 4; }
  f.key_mask = key_mask; f.km_sb = mask_batches == batch && batch > 1 ? seq : 0;
  return launch_flash_attention(f, s);
}

int af3_batch_diffusion_self_attention_forward(
    const uint16_t* q_data, const float* key_mask, int64_t mask_batches, const float* nonbatched_bias,
    int bias_quad_major, const uint16_t* w_qkvg, const float* query_b, int num_head,
    void* out, int out_dtype, int64_t batch, int64_t seq, int channels,
    void* workspace, size_t workspace_bytes, af3_stream_t stream) {
  int rc = self_attention_args_ok(q_data, key_mask, mask_batches, bias_quad_major, w_qkvg, out, out_dtype, num_head,
                                  batch, seq, channels);
  if (rc) return rc;
  Carver ws(workspace, workspace_bytes);
  bf16_t* qkvg = ws.take<bf16_t>((size_t)batch * seq * 4 * channels);
  if (!ws.ok) return AF3_ERR_WORKSPACE;
  return self_attention_run(q_data, key_mask, mask_batches, nonbatched_bias, bias_quad_major, w_qkvg, query_b,
                            num_head, out, out_dtype, batch, seq, channels, qkvg, static_cast<hipStream_t>(stream));
}

int af3_batch_diffusion_self_attention_forward_static(
    const uint16_t* q_data, const float* key_mask, int64_t mask_batches, const float* nonbatched_bias,
    int bias_quad_major, const uint16_t* w_qkvg, const float* query_b, int num_head,
    void* out, int out_dtype, int64_t batch, int64_t seq, int channels, af3_stream_t stream) {
  int rc = self_attention_args_ok(q_data, key_mask, mask_batches, bias_quad_major, w_qkvg, out, out_dtype, num_head,
                                  batch, seq, channels);
  if (rc) return rc;
  const size_t need = align_up((size_t)batch * seq * 4 * channels * sizeof(bf16_t), 256);
  if (need > STATIC_SCRATCH_BYTES) return AF3_ERR_TOO_LARGE;
  bf16_t* qkvg = static_cast<bf16_t*>(static_scratch_ptr());
  if (!qkvg) return AF3_ERR_LAUNCH;
  // The q/k/v/gate product writes every element of [batch * seq][4 * channels] before the attention kernel reads
  // any of them, so nothing left in the array by an earlier (possibly larger) call is ever read: no clearing.
  return self_attention_run(q_data, key_mask, mask_batches, nonbatched_bias, bias_quad_major, w_qkvg, query_b,
                            num_head, out, out_dtype, batch, seq, channels, qkvg, static_cast<hipStream_t>(stream));
}

// ---------------------------------------------------- masked row softmax, narrow fp32 layers
int af3_masked_softmax_rows_forward(const float* logits, const float* key_mask, uint16_t* out, int64_t rows,
                                    int64_t cols, int64_t out_ld, af3_stream_t stream) {
  if (cols <= 0 || cols > 0x7fffffff) return AF3_ERR_BAD_ARG;
  return launch_softmax_rows(logits, key_mask, out, rows, (int)cols, out_ld, static_cast<hipStream_t>(stream));
}

int af3_narrow_linear_f32_forward(const float* x, const float* w, const float* residual, float* y, int64_t rows,
                                  int k, int n_out, int relu_input, af3_stream_t stream) {
  return launch_narrow_linear_f32(x, w, residual, y, rows, k, n_out, relu_input, static_cast<hipStream_t>(stream));
}

int af3_atom_pair_cond_forward(const float* row, const float* col, const float* token_pair, const int32_t* query_token,
                               const int32_t* key_token, int64_t n_token, const float* query_pos, const float* key_pos,
                               const int32_t* query_uid, const int32_t* key_uid, const float* w_offsets,
                               const float* w_distances, const float* w_valid, const float* w_mlp1, const float* w_mlp2,
                               const float* w_mlp3, float* out, int64_t subsets, int64_t queries, int64_t keys,
                               af3_stream_t stream) {
  if (queries > 0x7fffffff || keys > 0x7fffffff || n_token > 0x7fff) return AF3_ERR_BAD_ARG;
  return launch_atom_pair_cond(row, col, token_pair, query_token, key_token, (int)n_token, query_pos, key_pos, query_uid,
                               key_uid, w_offsets, w_distances, w_valid, w_mlp1, w_mlp2, w_mlp3, out, subsets, (int)queries,
                               (int)keys, static_cast<hipStream_t>(stream));
}

int af3_atom_pair_logits_forward(const float* pair_cond, const float* ln_w, const float* w, float* out, int64_t subsets,
                                 int64_t queries, int64_t keys, int num_blocks, int num_head, af3_stream_t stream) {
  if (queries <= 0 || keys <= 0) return AF3_ERR_BAD_ARG;
  return launch_atom_pair_logits(pair_cond, ln_w, w, out, subsets, queries * keys, num_blocks, num_head,
                                 static_cast<hipStream_t>(stream));
}

int af3_pair_cond_init_forward(const void* pair, int pair_dtype, float in_scale, const int32_t* asym_id,
                               const int32_t* residue_index, const int32_t* token_index, const int32_t* entity_id,
                               const int32_t* sym_id, int max_relative_idx, int max_relative_chain, const float* ln_w,
                               const uint16_t* w_pair, const float* g_hot, const float* g_sum, float* out, int64_t n,
                               af3_stream_t stream) {
  if (bad_dtype(pair_dtype) || n <= 0 || n > 0x7fff) return AF3_ERR_BAD_ARG;
  PairCondInitArgs a;
  a.pair = pair; a.io_f32 = pair_dtype == AF3_F32; a.N = (int)n; a.in_scale = in_scale;
  a.asym_id = asym_id; a.residue_index = residue_index; a.token_index = token_index; a.entity_id = entity_id;
  a.sym_id = sym_id;
  a.max_rel_idx = max_relative_idx; a.max_rel_chain = max_relative_chain;
  a.n_rel = 4 * max_relative_idx + 2 * max_relative_chain + 7;
  a.ln_w = ln_w; a.w_pair = w_pair; a.g_hot = g_hot; a.g_sum = g_sum; a.out = out;
  return launch_pair_cond_init(a, static_cast<hipStream_t>(stream));
}

// -------------------------------------------------------------------- transpose
int af3_transpose_bf16_forward(const uint16_t* in, uint16_t* out, int64_t rows, int64_t cols, af3_stream_t stream) {
  return launch_transpose(in, out, rows, cols, static_cast<hipStream_t>(stream));
}

// ------------------------------------------------ atoms -> tokens aggregation
int af3_gathered_relu_mean_forward(const uint16_t* src, const int32_t* idx, const float* count, float* out,
                                   int64_t batch, int64_t n_src, int64_t n_out, int slots, int channels,
                                   af3_stream_t stream) {
  return launch_gathered_relu_mean(src, idx, count, out, batch, n_src, n_out, slots, channels,
                                   static_cast<hipStream_t>(stream));
}

int af3_atom_position_features_forward(const float* positions, const int32_t* rows, const float* weight,
                                       const float* cond, void* out, int out_dtype, int64_t batch, int64_t n_slots,
                                       int64_t n_queries, int channels, af3_stream_t stream) {
  if (bad_dtype(out_dtype)) return AF3_ERR_BAD_ARG;
  return launch_atom_position_features(positions, rows, weight, cond, out, out_dtype == AF3_F32, batch, n_slots,
                                       n_queries, channels, static_cast<hipStream_t>(stream));
}

int af3_gather_rows_add_forward(const uint16_t* src, const int32_t* rows, const uint16_t* add, uint16_t* out,
                                int64_t batch, int64_t n_src, int64_t n_queries, int channels, af3_stream_t stream) {
  return launch_gather_rows_add(src, rows, add, out, batch, n_src, n_queries, channels,
                                static_cast<hipStream_t>(stream));
}

int af3_position_update_forward(const uint16_t* x, const int32_t* rows, const float* ln_weight, const float* weight,
                                float* out, int64_t batch, int64_t n_src, int64_t n_out, int channels,
                                af3_stream_t stream) {
  return launch_ln_project3_gather(x, rows, ln_weight, weight, out, batch, n_src, n_out, channels,
                                   static_cast<hipStream_t>(stream));
}

// ------------------------------------------------------------ batched NT product
int af3_batched_nt_product_forward(
    const uint16_t* a, const uint16_t* b, uint16_t* c, int64_t batch, int64_t m, int64_t n, int64_t k,
    af3_stream_t stream) {
  if (!a || !b || !c || batch <= 0 || m <= 0 || n <= 0 || k <= 0 || (k & 7)) return AF3_ERR_BAD_ARG;
  if (m > 0x7fffffff || n > 0x7fffffff || k > 0x7fffffff || batch > 0x7fffffff) return AF3_ERR_BAD_ARG;
  GemmArgs g;
  g.A = a; g.B = b; g.C = c;
  g.M = (int)m; g.N = (int)n; g.K = (int)k; g.batch = (int)batch;
  g.lda = g.ldb = k; g.ldc = n;
  g.sA = m * k; g.sB = n * k; g.sC = m * n;
  return contraction(g, static_cast<hipStream_t>(stream));
}

// --------------------------------------------------- windowed (atom) cross-attention
size_t af3_batch_diffusion_cross_attention_workspace_bytes(int64_t batch, int64_t sq, int64_t sk, int channels) {
  if (batch <= 0 || sq <= 0 || sk <= 0 || channels <= 0) return 0;
  return align_up((size_t)batch * sq * 2 * channels * sizeof(bf16_t), 256) +
         align_up((size_t)batch * sk * 2 * channels * sizeof(bf16_t), 256);
}

int af3_batch_diffusion_cross_attention_forward(
    const uint16_t* q_data, const uint16_t* m_data,
    const float* pair_logits, const float* mask_q, const float* mask_k, int64_t bias_batches,
    const uint16_t* w_qg, const uint16_t* w_kv, const float* query_b, int num_head,
    void* out, int out_dtype, int64_t batch, int64_t sq, int64_t sk, int channels,
    void* workspace, size_t workspace_bytes, af3_stream_t stream) {
  if (!q_data || !m_data || !w_qg || !w_kv || !out) return AF3_ERR_BAD_ARG;
  if (bad_dtype(out_dtype) || batch <= 0 || sq <= 0 || sk <= 0 || channels <= 0 || (channels & 7) ||
      num_head <= 0 || channels % num_head)
    return AF3_ERR_BAD_ARG;
  if ((mask_q == nullptr) != (mask_k == nullptr)) return AF3_ERR_BAD_ARG;
  if ((pair_logits || mask_q) && (bias_batches <= 0 || batch % bias_batches)) return AF3_ERR_BAD_ARG;
  if (batch * sq > 0x7fffffff || batch * sk > 0x7fffffff) return AF3_ERR_BAD_ARG;
  const int d = channels / num_head;
  if (d != 24 && d != 32 && d != 48) return AF3_ERR_UNSUPPORTED;
  Carver ws(workspace, workspace_bytes);
  bf16_t* qg = ws.take<bf16_t>((size_t)batch * sq * 2 * channels);
  bf16_t* kv = ws.take<bf16_t>((size_t)batch * sk * 2 * channels);
  if (!ws.ok) return AF3_ERR_WORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);

  GemmArgs g;
  g.A = q_data; g.B = w_qg; g.C = qg;
  g.M = (int)(batch * sq); g.N = 2 * channels; g.K = channels;
  g.lda = channels; g.ldb = channels; g.ldc = 2 * channels;
  g.epi = EPI_SEGMENTED; g.seg_len = channels;
  g.seg_ops = SEG_BIAS_SCALE | (SEG_SIGMOID << 4);
  g.alpha = 1.0f / sqrtf((float)d);
  g.bias = query_b; g.bias_len = channels;  // the query segment's columns only
  int rc = launch_gemm_nt(g, s);
  if (rc) return rc;
  GemmArgs g2;
  g2.A = m_data; g2.B = w_kv; g2.C = kv;
  g2.M = (int)(batch * sk); g2.N = 2 * channels; g2.K = channels;
  g2.lda = channels; g2.ldb = channels; g2.ldc = 2 * channels;
  rc = launch_gemm_nt(g2, s);
  if (rc) return rc;

  FlashArgs f;
  f.q = qg; f.g = qg + channels; f.k = kv; f.v = kv + channels;
  f.q_ss = f.g_ss = f.k_ss = f.v_ss = 2 * channels;
  f.q_sb = f.g_sb = sq * 2 * channels;
  f.k_sb = f.v_sb = sk * 2 * channels;
  f.out = out; f.out_f32 = out_dtype == AF3_F32; f.o_ss = channels; f.o_sb = sq * channels;
  f.B = (int)batch; f.H = num_head; f.Sq = (int)sq; f.Sk = (int)sk; f.d = d;
  f.bias = pair_logits; f.bias_sb = (int64_t)num_head * sq * sk; f.bias_sh = sq * sk; f.bias_sq = sk;
  f.qpad = mask_q; f.kpad = mask_k; f.qp_sb = sq; f.kp_sb = sk;
  f.bias_mod = (pair_logits || mask_q) ? (int)bias_batches : 0;
  return launch_flash_attention(f, s);
}

size_t af3_gathered_cross_attention_workspace_bytes(int64_t batch, int64_t sq, int64_t samples, int64_t n_atoms,
                                                    int channels) {
  if (batch <= 0 || sq <= 0 || samples <= 0 || n_atoms <= 0 || channels <= 0) return 0;
  return align_up((size_t)batch * sq * 2 * channels * sizeof(bf16_t), 256) +
         align_up((size_t)samples * n_atoms * 2 * channels * sizeof(bf16_t), 256);
}

int af3_gathered_cross_attention_forward(
    const uint16_t* q_data, const uint16_t* atom_data, const int32_t* key_rows,
    const float* pair_logits, const float* mask_q, const float* mask_k, int64_t bias_batches,
    const uint16_t* w_qg, const uint16_t* w_kv, const float* query_b, int num_head,
    void* out, int out_dtype, int64_t batch, int64_t sq, int64_t sk, int64_t samples, int64_t n_atoms, int channels,
    void* workspace, size_t workspace_bytes, af3_stream_t stream) {
  if (!q_data || !atom_data || !key_rows || !w_qg || !w_kv || !out) return AF3_ERR_BAD_ARG;
  if (bad_dtype(out_dtype) || batch <= 0 || sq <= 0 || sk <= 0 || samples <= 0 || n_atoms <= 0 || channels <= 0 ||
      (channels & 7) || num_head <= 0 || channels % num_head)
    return AF3_ERR_BAD_ARG;
  if ((mask_q == nullptr) != (mask_k == nullptr)) return AF3_ERR_BAD_ARG;
  if (bias_batches <= 0 || batch != samples * bias_batches) return AF3_ERR_BAD_ARG;
  if (batch * sq > 0x7fffffff || samples * n_atoms > 0x7fffffff) return AF3_ERR_BAD_ARG;
  const int d = channels / num_head;
  if (d != 24 && d != 32 && d != 48) return AF3_ERR_UNSUPPORTED;
  Carver ws(workspace, workspace_bytes);
  bf16_t* qg = ws.take<bf16_t>((size_t)batch * sq * 2 * channels);
  bf16_t* kv = ws.take<bf16_t>((size_t)samples * n_atoms * 2 * channels);
  if (!ws.ok) return AF3_ERR_WORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);

  GemmArgs g;
  g.A = q_data; g.B = w_qg; g.C = qg;
  g.M = (int)(batch * sq); g.N = 2 * channels; g.K = channels;
  g.lda = channels; g.ldb = channels; g.ldc = 2 * channels;
  g.epi = EPI_SEGMENTED; g.seg_len = channels;
  g.seg_ops = SEG_BIAS_SCALE | (SEG_SIGMOID << 4);
  g.alpha = 1.0f / sqrtf((float)d);
  g.bias = query_b; g.bias_len = channels;  // the query segment's columns only
  int rc = launch_gemm_nt(g, s);
  if (rc) return rc;
  GemmArgs g2;
  g2.A = atom_data; g2.B = w_kv; g2.C = kv;
  g2.M = (int)(samples * n_atoms); g2.N = 2 * channels; g2.K = channels;
  g2.lda = channels; g2.ldb = channels; g2.ldc = 2 * channels;
  rc = launch_gemm_nt(g2, s);
  if (rc) return rc;

  FlashArgs f;
  f.q = qg; f.g = qg + channels; f.k = kv; f.v = kv + channels;
  f.q_ss = f.g_ss = f.k_ss = f.v_ss = 2 * channels;
  f.q_sb = f.g_sb = sq * 2 * channels;
  f.k_sb = f.v_sb = n_atoms * 2 * channels;   // one K / V table per sample
  f.key_rows = key_rows;
  f.out = out; f.out_f32 = out_dtype == AF3_F32; f.o_ss = channels; f.o_sb = sq * channels;
  f.B = (int)batch; f.H = num_head; f.Sq = (int)sq; f.Sk = (int)sk; f.d = d;
  f.bias = pair_logits; f.bias_sb = (int64_t)num_head * sq * sk; f.bias_sh = sq * sk; f.bias_sq = sk;
  f.qpad = mask_q; f.kpad = mask_k; f.qp_sb = sq; f.kp_sb = sk;
  f.bias_mod = (int)bias_batches;
  return launch_flash_attention(f, s);
}

// ------------------------------------------------------------------ pair logits
int af3_pair_logits_forward(
    const void* pair, int io_dtype, const float* norm_weight, const float* norm_bias,
    const uint16_t* w, int n_out, float* out, int64_t n, af3_stream_t stream) {
  if (!pair || !w || !out || !norm_weight) return AF3_ERR_BAD_ARG;
  if (bad_dtype(io_dtype) || n <= 0 || n > 8192 || n_out <= 0) return AF3_ERR_BAD_ARG;
  AttnProjArgs p;
  p.pair = pair; p.io_f32 = io_dtype == AF3_F32; p.N = (int)n;
  p.ln_w = norm_weight; p.ln_b = norm_bias;
  p.w_bias = w; p.n_bias = n_out; p.out_bias = out;
  return launch_attn_proj(p, static_cast<hipStream_t>(stream));
}

// ------------------------------------------------------------------- row norm
int af3_layer_norm_forward(
    const void* x, int x_dtype, uint16_t* y, int64_t rows, int channels,
    const float* weight, const float* bias, const float* scale, const float* shift,
    int64_t cond_rows, int64_t cond_ld, af3_stream_t stream) {
  if (!x || !y || bad_dtype(x_dtype)) return AF3_ERR_BAD_ARG;
  RowNormArgs a;
  a.x = x; a.x_f32 = x_dtype == AF3_F32; a.y = y; a.rows = rows; a.ldx = a.ldy = channels; a.C = channels;
  a.weight = weight; a.bias = bias; a.scale = scale; a.shift = shift;
  a.cond_rows = cond_rows; a.ld_cond = cond_ld;
  return launch_row_norm(a, static_cast<hipStream_t>(stream));
}

// --------------------------------------------------------------------- linear
int af3_linear_forward(
    const uint16_t* x, const uint16_t* w, const float* bias, void* y, int y_dtype,
    int64_t m, int n, int k, int mode, float alpha, int sigmoid,
    const float* gate, int64_t gate_rows, int64_t gate_ld, const void* residual, int res_dtype, af3_stream_t stream) {
  if (!x || !w || !y || bad_dtype(y_dtype) || m <= 0 || m > 0x7fffffff || n <= 0 || k <= 0) return AF3_ERR_BAD_ARG;
  if (gate_ld != 0 && gate_ld < n) return AF3_ERR_BAD_ARG;
  if (mode != AF3_LINEAR_PLAIN && mode != AF3_LINEAR_SWIGLU && mode != AF3_LINEAR_GATE_RES &&
      mode != AF3_LINEAR_REGROUP32 && mode != AF3_LINEAR_ROWGATE_RES)
    return AF3_ERR_BAD_ARG;
  if (residual && bad_dtype(res_dtype)) return AF3_ERR_BAD_ARG;
  GemmArgs g;
  if (mode == AF3_LINEAR_REGROUP32) {
    if ((m & 31) || (n & 31) || gate || residual) return AF3_ERR_BAD_ARG;
    g.regroup32 = 1;
    mode = AF3_LINEAR_PLAIN;
  }
  if (mode == AF3_LINEAR_ROWGATE_RES) {
    if (!gate || gate_rows <= 0) return AF3_ERR_BAD_ARG;
    g.gate_per_row = 1;
    mode = AF3_LINEAR_GATE_RES;
  }
  g.A = x; g.B = w; g.C = y;
  g.M = (int)m; g.N = n; g.K = k;
  g.lda = k; g.ldb = k;
  g.ldc = mode == AF3_LINEAR_SWIGLU ? n / 2 : n;
  g.out_f32 = y_dtype == AF3_F32;
  g.epi = mode; g.alpha = alpha; g.bias = bias; g.bias_len = n; g.act_sigmoid = sigmoid;
  g.gate = gate; g.gate_rows = (int)gate_rows; g.ld_gate = gate_ld ? gate_ld : n;
  if (residual) {
    if (res_dtype == AF3_F32) g.res_f32 = static_cast<const float*>(residual);
    else g.res_bf16 = static_cast<const bf16_t*>(residual);
    g.ld_res = n;
  }
  return launch_gemm_nt(g, static_cast<hipStream_t>(stream));
}

// ----------------------------------------------------------------- diagnostics
int af3_linear_bias_span(int64_t m, int n, int k, int seg_len, int seg_ops, int64_t* first, int64_t* last) {
  if (!first || !last || m <= 0 || m > 0x7fffffff || n <= 0 || k <= 0 || seg_len < 0) return AF3_ERR_BAD_ARG;
  if (seg_len > 0 && ((seg_len & 7) || n > 8 * seg_len)) return AF3_ERR_BAD_ARG;
  // the product as af3_linear_forward (seg_len = 0) or the segmented projections (seg_len > 0) describe
  // it; the operand pointers only have to look aligned, nothing is dereferenced
  GemmArgs g;
  g.A = reinterpret_cast<const bf16_t*>(uintptr_t(16)); g.B = g.A; g.C = reinterpret_cast<void*>(uintptr_t(16));
  g.bias = reinterpret_cast<const float*>(uintptr_t(16));
  g.M = (int)m; g.N = n; g.K = k; g.lda = g.ldb = k; g.ldc = n;
  if (seg_len > 0) { g.epi = EPI_SEGMENTED; g.seg_len = seg_len; g.seg_ops = seg_ops; }
  gemm_bias_span(g, gemm_big_tile_choice(g) >= 0, first, last);
  return AF3_OK;
}

// ------------------------------------------------------- kernel-level entry points
int af3_triangle_contraction_forward(
    const uint16_t* a, const uint16_t* b, uint16_t* t, int64_t n, af3_stream_t stream) {
  if (!a || !b || !t || n <= 0 || n > 8192) return AF3_ERR_BAD_ARG;
  const int64_t np = pad8(n);
  GemmArgs g;
  g.A = a; g.B = b; g.C = t;
  g.M = g.N = (int)n; g.K = (int)np; g.batch = C_PAIR;
  g.lda = g.ldb = g.ldc = np;
  g.sA = g.sB = g.sC = n * np;
  return contraction(g, static_cast<hipStream_t>(stream));
}

int af3_grid_attention_core_forward(
    const uint16_t* q, const uint16_t* k, const uint16_t* vt,
    const uint16_t* pair_bias, const float* mask, uint16_t* og, int64_t n, af3_stream_t stream) {
  if (n <= 0 || n > 8192) return AF3_ERR_BAD_ARG;
  TriAttnArgs t;
  t.q = q; t.k = k; t.vt = vt; t.bias = pair_bias; t.mask = mask; t.og = og;
  t.N = (int)n; t.ldn = tri_ldn(n);
  return launch_triattn_flash(t, static_cast<hipStream_t>(stream));
}

// ------------------------------------------------------------- fp32 check mode
int af3_check_gemm_f32(
    const float* a, const float* b, float* c, int64_t m, int64_t n, int64_t k, int64_t batch,
    int64_t lda, int64_t ka, int64_t ldb, int64_t kb, int64_t ldc, int64_t sa, int64_t sb, int64_t sc,
    const float* bias, float alpha, int sigmoid, const float* mul, int64_t mul_rows, int64_t ld_mul,
    const float* add, int64_t ld_add, int64_t s_add, af3_stream_t stream) {
  if (m > 0x7fffffff || n > 0x7fffffff || k > 0x7fffffff || batch > 65535) return AF3_ERR_BAD_ARG;
  CkGemmArgs g;
  g.A = a; g.B = b; g.C = c; g.M = (int)m; g.N = (int)n; g.K = (int)k; g.batch = (int)batch;
  g.lda = lda; g.ka = ka; g.ldb = ldb; g.kb = kb; g.ldc = ldc; g.sA = sa; g.sB = sb; g.sC = sc;
  g.bias = bias; g.alpha = alpha; g.sigmoid = sigmoid;
  g.mul = mul; g.mul_rows = mul_rows; g.ld_mul = ld_mul; g.add = add; g.ld_add = ld_add; g.s_add = s_add;
  return launch_ck_gemm(g, static_cast<hipStream_t>(stream));
}

int af3_check_layer_norm_f32(
    const float* x, float* y, int64_t rows, int channels, const float* weight, const float* bias,
    const float* scale, const float* shift, int64_t cond_rows, int64_t cond_ld, af3_stream_t stream) {
  CkNormArgs a;
  a.x = x; a.y = y; a.rows = rows; a.C = channels; a.weight = weight; a.bias = bias;
  a.scale = scale; a.shift = shift; a.cond_rows = cond_rows; a.ld_cond = cond_ld;
  return launch_ck_norm(a, static_cast<hipStream_t>(stream));
}

int af3_check_elementwise_f32(
    int op, const float* x0, const float* x1, const float* x2, float* y0, float* y1,
    int64_t n0, int64_t n1, int flag, af3_stream_t stream) {
  return launch_ck_elementwise(op, x0, x1, x2, y0, y1, n0, n1, flag, static_cast<hipStream_t>(stream));
}

int af3_check_attention_f32(
    const float* q, const float* k, const float* v, float* out,
    int64_t q_sb, int64_t q_ss, int64_t k_sb, int64_t k_ss, int64_t v_sb, int64_t v_ss, int64_t o_sb, int64_t o_ss,
    int64_t batch, int num_head, int64_t sq, int64_t sk, int head_dim,
    const float* bias, int64_t bias_sb, int64_t bias_sh, int64_t bias_sq, int64_t bias_sk, int64_t bias_mod,
    const float* key_mask, int64_t km_sb, const float* qpad, const float* kpad, af3_stream_t stream) {
  if (batch > 0x7fffffff || sq > 0x7fffffff || sk > 0x7fffffff || bias_mod > 0x7fffffff) return AF3_ERR_BAD_ARG;
  CkAttnArgs a;
  a.q = q; a.k = k; a.v = v; a.out = out;
  a.q_sb = q_sb; a.q_ss = q_ss; a.k_sb = k_sb; a.k_ss = k_ss; a.v_sb = v_sb; a.v_ss = v_ss; a.o_sb = o_sb; a.o_ss = o_ss;
  a.B = (int)batch; a.H = num_head; a.Sq = (int)sq; a.Sk = (int)sk; a.d = head_dim;
  a.bias = bias; a.bias_sb = bias_sb; a.bias_sh = bias_sh; a.bias_sq = bias_sq; a.bias_sk = bias_sk;
  a.bias_mod = (int)bias_mod; a.key_mask = key_mask; a.km_sb = km_sb; a.qpad = qpad; a.kpad = kpad;
  return launch_ck_attention(a, static_cast<hipStream_t>(stream));
}

}  // extern "C"
