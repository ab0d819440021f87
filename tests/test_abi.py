"""CPU-side checks of the boundary: the shared library loads and exports every
symbol include/af3_hip.h declares, the ctypes table matches the header, and the
host-side weight packing / module plumbing behaves (no GPU compute)."""

import ctypes
import os
import re

import pytest
import torch

from oracle import af3_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "af3_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(af3_[a-z0-9_]+)\s*\(", text)))


def header_abi_version():
    return int(re.search(r"#define\s+AF3_ABI_VERSION\s+(\d+)", open(HEADER).read()).group(1))


def count_params(name):
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    m = re.search(r"\b%s\s*\((.*?)\)\s*;" % re.escape(name), text, flags=re.S)
    args = m.group(1).strip()
    return 0 if args in ("", "void") else args.count(",") + 1


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for required in ("af3_triangle_multiplication_forward", "af3_grid_self_attn_forward",
                     "af3_transition_forward", "af3_batch_diffusion_self_attention_forward",
                     "af3_batch_diffusion_cross_attention_forward"):
        assert required in syms


def test_library_exports_every_declared_symbol(pkg):
    if not os.path.exists(pkg.lib.LIB_PATH):
        pytest.fail("libaf3hip.so is not built: run __graft_entry__.build()")
    lib = ctypes.CDLL(pkg.lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} declared in af3_hip.h but not exported"


def test_ctypes_table_matches_header(pkg):
    assert sorted(pkg.lib.SIGNATURES) == declared_symbols()
    for name, (_, args) in pkg.lib.SIGNATURES.items():
        assert len(args) == count_params(name), name


def test_error_strings_and_version(pkg):
    lib = pkg.lib.load()
    # the library reports the version its header declares
    assert lib.af3_abi_version() == header_abi_version() == 2
    assert lib.af3_error_string(0) == b"ok"
    assert b"workspace" in lib.af3_error_string(-2)
    with pytest.raises(pkg.lib.Af3Error):
        pkg.lib.check(-1, "x")


def test_workspace_queries(pkg):
    lib = pkg.lib.load()
    n = 100
    np_ = 104
    assert lib.af3_triangle_multiplication_workspace_bytes(n) >= 3 * 128 * n * np_ * 2
    # q, k, v^T and the attention output (bf16) + the four fp16 bias heads
    assert lib.af3_grid_self_attn_workspace_bytes(n, 4) >= n * n * (4 * 128 * 2 + 4 * 2)
    assert lib.af3_triangle_multiplication_workspace_bytes(0) == 0


def test_null_and_bad_arguments_are_rejected_without_a_gpu(pkg):
    """Argument validation happens before any launch, so it can run here."""
    lib = pkg.lib.load()
    assert lib.af3_transition_forward(None, 0, None, None, None, None, 512, None, 0, 10, None) == -1
    assert lib.af3_linear_forward(None, None, None, None, 0, 1, 8, 8, 0, 1.0, 0, None, 0, 0, None, 0, None) == -1
    assert lib.af3_triangle_multiplication_forward(None, 0, None, 0, None, None, None, None, None, None, None,
                                                   None, 0, 8, None, 0, None) == -1


def _bias_span(lib, m, n, k, seg_len=0, seg_ops=0):
    first, last = ctypes.c_int64(-1), ctypes.c_int64(-1)
    assert lib.af3_linear_bias_span(m, n, k, seg_len, seg_ops, ctypes.byref(first), ctypes.byref(last)) == 0
    return first.value, last.value


def test_bias_entries_a_launch_reads_stay_inside_the_callers_array(pkg):
    """The dense kernels fetch the column bias in groups; the launch path refuses a product whose groups
    would reach past the extent the caller vouches for.  The span comes from the formula the device
    code takes its addresses from.  Shapes: the q-k-v-gate projection of
    tests/test_gpu_big_tile.py::test_self_attention_projection_segments (5 x 768 tokens, 768 channels:
    the 256x256 tile; its bias covers the 768 query columns only), one sample of it (128x128 tile),
    and plain biased products with ragged column counts on both tiles."""
    lib = pkg.lib.load()
    BIAS_SCALE, PLAIN, SIGMOID = 1, 0, 2
    qkvg = BIAS_SCALE | (PLAIN << 4) | (PLAIN << 8) | (SIGMOID << 12)
    for m in (5 * 768, 768):                       # large tile / small tile
        assert _bias_span(lib, m, 4 * 768, 768, 768, qkvg) == (0, 768)
    # queries and gates of the atom cross-attention: 2 x 128 columns, bias for the first 128
    assert _bias_span(lib, 5 * 576 * 32, 256, 128, 128, BIAS_SCALE | (SIGMOID << 4)) == (0, 128)
    # a biased segment further right reaches further: the launch path compares this with the extent
    assert _bias_span(lib, 5 * 768, 4 * 768, 768, 768, PLAIN | (BIAS_SCALE << 8)) == (2 * 768, 3 * 768)
    # unsegmented: exactly the n columns, whatever the tile and however ragged n is
    for m, n, k in ((3850, 2824, 200), (5000, 3400, 72), (300, 2824, 200), (100, 40, 64), (4096, 2560, 768)):
        assert _bias_span(lib, m, n, k) == (0, n), (m, n, k)
    # no segment uses the bias: nothing is read
    first, last = _bias_span(lib, 5 * 768, 4 * 768, 768, 768, PLAIN | (SIGMOID << 12))
    assert first == last
    assert lib.af3_linear_bias_span(0, 8, 8, 0, 0, None, None) == -1


def test_gathered_cross_attention_and_regrouped_store_reject_bad_arguments(pkg):
    lib = pkg.lib.load()
    one = 1 << 20     # a non-null dummy address: every check below fails before it is touched
    args = dict(q=one, atoms=one, rows=one, pl=None, mq=None, mk=None, bb=4, wqg=one, wkv=one, qb=None, h=4,
                out=one, dt=0, batch=8, sq=32, sk=128, samples=2, n_atoms=128, c=128, ws=one, wsb=1 << 30, st=None)

    def call(**kw):
        a = dict(args, **kw)
        return lib.af3_gathered_cross_attention_forward(
            a["q"], a["atoms"], a["rows"], a["pl"], a["mq"], a["mk"], a["bb"], a["wqg"], a["wkv"], a["qb"], a["h"],
            a["out"], a["dt"], a["batch"], a["sq"], a["sk"], a["samples"], a["n_atoms"], a["c"], a["ws"], a["wsb"],
            a["st"])
    assert call(rows=None) == -1                       # key_rows is required
    assert call(batch=9) == -1                         # batch must be samples * bias_batches
    assert call(mq=one) == -1                          # masks come in pairs
    assert call(c=100) == -1                           # channels: multiple of 8 and of the head count
    assert call(h=8) != 0                              # head dim 16 is not supported
    assert call(wsb=16) == -2                          # workspace too small
    assert lib.af3_gathered_cross_attention_workspace_bytes(8, 32, 2, 128, 128) >= (8 * 32 + 2 * 128) * 256 * 2
    # regrouped store: rows of both operands in multiples of 32, no gate / residual
    assert lib.af3_linear_forward(one, one, None, one, 0, 48, 64, 8, 4, 1.0, 0, None, 0, 0, None, 0, None) == -1
    assert lib.af3_linear_forward(one, one, None, one, 0, 64, 64, 8, 4, 1.0, 0, one, 1, 0, None, 0, None) == -1
    assert lib.af3_linear_forward(one, one, None, one, 0, 64, 64, 8, 5, 1.0, 0, None, 0, 0, None, 0, None) == -1   # row gate missing
    assert lib.af3_linear_forward(one, one, None, one, 0, 64, 64, 8, 6, 1.0, 0, None, 0, 0, None, 0, None) == -1   # unknown mode
    assert lib.af3_linear_forward(one, one, None, one, 0, 64, 64, 8, 3, 1.0, 0, one, 1, 32, None, 0, None) == -1  # gate rows overlap


def test_quad_major_bias_layout_and_its_argument_check(pkg):
    """[H, Sq, Sk] -> [H, Sk/4, Sq, 4]: element (h, q, k) at ((h * Sk/4 + k/4) * Sq + q) * 4 + k%4."""
    bias = torch.arange(2 * 6 * 8, dtype=torch.float32).reshape(2, 6, 8)
    qm = pkg.ops.quad_major_bias(bias)
    assert qm.shape == (2, 2, 6, 4) and qm.is_contiguous()
    flat = qm.reshape(-1)
    for h, q, k in ((0, 0, 0), (1, 5, 7), (0, 3, 4), (1, 2, 1)):
        assert flat[((h * 2 + k // 4) * 6 + q) * 4 + k % 4] == bias[h, q, k]
    with pytest.raises(ValueError):
        pkg.ops.quad_major_bias(torch.zeros(2, 6, 6))
    lib = pkg.lib.load()
    one = 1 << 20
    # quad-major bias with a sequence length that is not a multiple of 4, or an unknown layout flag
    assert lib.af3_batch_diffusion_self_attention_forward(one, None, 1, one, 1, one, None, 4, one, 0, 1, 30, 128,
                                                          one, 1 << 30, None) == -1
    assert lib.af3_batch_diffusion_self_attention_forward(one, None, 1, one, 2, one, None, 4, one, 0, 1, 32, 128,
                                                          one, 1 << 30, None) == -1


def test_gathered_relu_mean_rejects_bad_arguments(pkg):
    lib = pkg.lib.load()
    one = 1 << 20
    assert lib.af3_gathered_relu_mean_forward(one, None, one, one, 1, 8, 8, 4, 128, None) == -1    # no index table
    assert lib.af3_gathered_relu_mean_forward(one, one, one, one, 1, 8, 8, 33, 128, None) == -1    # too many slots
    assert lib.af3_gathered_relu_mean_forward(one, one, one, one, 1, 8, 8, 4, 100, None) == -1     # channels % 8
    assert lib.af3_gathered_relu_mean_forward(one + 2, one, one, one, 1, 8, 8, 4, 128, None) == -1  # misaligned
    assert lib.af3_atom_position_features_forward(one, None, one, one, one, 0, 1, 8, 8, 128, None) == -1   # no rows
    assert lib.af3_gather_rows_add_forward(one, one, None, one, 1, 8, 8, 128, None) == -1                   # no addend
    assert lib.af3_gather_rows_add_forward(one, one, one, one, 1, 8, 8, 100, None) == -1                    # channels % 8
    assert lib.af3_position_update_forward(one, one, one, one, one, 1, 8, 8, 64, None) != 0                  # channels != 128
    assert lib.af3_position_update_forward(one, None, one, one, one, 1, 8, 8, 128, None) == -1               # no rows
    assert lib.af3_atom_position_features_forward(one, one, one, one, one, 2, 1, 8, 8, 128, None) == -1    # dtype
    assert lib.af3_atom_position_features_forward(one, one, one, one, one, 0, 1, 8, 8, 100, None) == -1    # channels % 8


def test_conditioning_kernels_reject_bad_arguments(pkg):
    """The per-batch conditioning entry points of the diffusion head check their arguments before any launch."""
    lib = pkg.lib.load()
    one = 1 << 20
    ids = (one, one, one, one, one)
    ok_tail = (32, 2, one, one, one, one, one, 16, None)
    assert lib.af3_pair_cond_init_forward(None, 0, 1.0, *ids, *ok_tail) == -1                        # no pair tensor
    assert lib.af3_pair_cond_init_forward(one, 5, 1.0, *ids, *ok_tail) == -1                         # dtype
    assert lib.af3_pair_cond_init_forward(one, 0, 1.0, one, one, None, one, one, *ok_tail) == -1     # a token feature missing
    assert lib.af3_pair_cond_init_forward(one, 0, 1.0, *ids, 32, 2, one, one, one, one, one, 0, None) == -1    # n = 0
    assert lib.af3_pair_cond_init_forward(one + 4, 0, 1.0, *ids, *ok_tail) == -1                     # misaligned
    assert lib.af3_atom_pair_logits_forward(one, one, one, None, 4, 32, 128, 3, 4, None) == -1       # no output
    assert lib.af3_atom_pair_logits_forward(one, one, one, one, 4, 32, 128, 9, 4, None) != 0         # more than 32 planes
    assert lib.af3_atom_pair_logits_forward(one, one, one, one, 4, 0, 128, 3, 4, None) == -1         # no queries
    w = (one, one, one, one, one, one)
    assert lib.af3_atom_pair_cond_forward(one, None, None, None, None, 0, one, one, one, one, *w, one, 4, 32, 128, None) == -1
    assert lib.af3_atom_pair_cond_forward(one, one, one, None, one, 8, one, one, one, one, *w, one, 4, 32, 128, None) == -1  # token table missing
    assert lib.af3_atom_pair_cond_forward(one, one, None, None, None, 0, one, one, one, one, *w, one, 0, 32, 128, None) == -1


def test_new_modules_share_the_reference_parameter_names(pkg):
    from oracle import af3_head_oracle as H
    from oracle import af3_msa_oracle as M
    g = torch.Generator().manual_seed(0)
    pairs = [
        (pkg.nn.DiffusionHead(num_blocks=4), H.make_diffusion_head_params(g, num_blocks=4)),
        (pkg.nn.AtomCrossAttDecoder(), H.make_decoder_params(g)),
        (pkg.nn.AtomCrossAttEncoder(), H.make_encoder_params(g, 384, False, False, False)),
        (pkg.nn.EvoformerBlock(), M.make_evoformer_block_params(g)),
    ]
    for mod, params in pairs:
        assert sorted(mod.state_dict()) == sorted(params)
        for k, v in mod.state_dict().items():
            assert v.shape == params[k].shape, k
    mesh = object()
    assert pkg.nn.DistributeDiffusionHead(mesh, use_batch_infer=True).use_batch_infer is True
    assert pkg.nn.DistributeEvoformerBlock(mesh, c_msa=64, c_pair=128).c_msa == 64
    assert pkg.nn.DistributeAtomCrossAttDecoder(mesh, use_batch_infer=True).use_batch_infer is True
    assert pkg.nn.DistributeOuterProductMean(mesh, c_msa=64, num_output_channel=128).num_outer_channel == 32


def test_cpu_tensors_raise(pkg):
    with pytest.raises(ValueError):
        pkg.ops.layer_norm(torch.randn(4, 128))
    mod = pkg.nn.Transition(c_x=128)
    with pytest.raises(ValueError):
        mod(torch.randn(4, 128))


def test_pack_swiglu_and_pad_rows(pkg):
    from distributed_xfold_amd.nn.base import pack_swiglu, pad_rows
    hidden, c = 128, 8
    w = torch.arange(2 * hidden * c, dtype=torch.float32).reshape(2 * hidden, c)
    pk = pack_swiglu(w, 32)
    for blk in range(hidden // 32):
        assert torch.equal(pk[64 * blk: 64 * blk + 32], w[32 * blk: 32 * blk + 32])
        assert torch.equal(pk[64 * blk + 32: 64 * blk + 64], w[hidden + 32 * blk: hidden + 32 * blk + 32])
    padded = pad_rows(torch.ones(4, 8), 32)
    assert padded.shape == (32, 8) and padded[4:].abs().sum() == 0 and padded[:4].sum() == 32


def test_trimul_packing_matches_the_interleave(pkg):
    """Packed chunk layout: operand a of channel c is nn.Linear row 2c, operand b
    row 2c+1 (reference de-interleave, nn/d_triangle_multiplication.py:128-129)."""
    mod = pkg.nn.TriangleMultiplication()
    packed = mod.packed()["w_proj_gate"].float()
    wp = mod.projection.weight.detach().bfloat16().float()
    wg = mod.gate.weight.detach().bfloat16().float()
    for chunk in range(4):
        half, lo = chunk // 2, 64 * (chunk % 2)
        for r in (0, 17, 63):
            ch = lo + r
            assert torch.equal(packed[chunk, r], wp[2 * ch + half])
            assert torch.equal(packed[chunk, 64 + r], wg[2 * ch + half])


def test_modules_share_the_reference_parameter_names(pkg):
    g = torch.Generator().manual_seed(0)
    pairs = [
        (pkg.nn.PairformerBlock(), O.make_pairformer_block_params(g)),
        (pkg.nn.PairformerBlock(with_single=False), O.make_pairformer_block_params(g, with_single=False)),
        (pkg.nn.DiffusionTransformer(num_blocks=4), O.make_diffusion_transformer_params(g, num_blocks=4)),
        (pkg.nn.DiffusionCrossAttTransformer(), O.make_cross_att_transformer_params(g)),
        (pkg.nn.GridSelfAttention(), O.make_grid_self_attention_params(g)),
        (pkg.nn.TriangleMultiplication(), O.make_triangle_multiplication_params(g)),
        (pkg.nn.Transition(c_x=384), O.make_transition_params(g, 384)),
    ]
    for mod, params in pairs:
        assert sorted(mod.state_dict()) == sorted(params)
        for k, v in mod.state_dict().items():
            assert v.shape == params[k].shape, k


def test_reference_constructor_signatures(pkg):
    """The reference's distributed classes take a device mesh first
    (nn/d_attention.py:24, nn/d_primitives.py:23, nn/d_pairformer.py:37-47)."""
    mesh = object()
    nn = pkg.nn
    assert nn.DistributeGridSelfAttention(mesh, c_pair=128, num_head=4, transpose=True).transpose is True
    assert nn.DistributeTransition(mesh, c_x=384, num_intermediate_factor=4).c_x == 384
    assert nn.DistributeTransition(mesh, 128, 2).num_intermediate_factor == 2
    assert nn.XSMMTriangleMultiplication(c_pair=128, _outgoing=False).c_equation == "kjc,kic->ijc"
    blk = nn.DistributePairformerBlock(mesh, with_single=False)
    assert not hasattr(blk, "single_attention_")
    sa = nn.DistributeSelfAttention(mesh, c_x=384, num_head=16, use_single_cond=False, use_batch_infer=False)
    assert sa.qkv_dim == 24
    assert hasattr(sa, "load_xsmm_params") and hasattr(sa, "xsmm_forward")


def test_library_is_not_older_than_its_sources(pkg):
    """A stale libaf3hip.so (sources edited, library not rebuilt) would make the
    ctypes table and the binary disagree about argument lists."""
    csrc = os.path.join(os.path.dirname(pkg.lib.LIB_PATH), "csrc")
    so_time = os.path.getmtime(pkg.lib.LIB_PATH)
    srcs = [os.path.join(csrc, f) for f in os.listdir(csrc) if f.endswith((".hip", ".h"))] + [HEADER]
    stale = [os.path.basename(f) for f in srcs if os.path.getmtime(f) > so_time + 1]
    assert not stale, f"rebuild libaf3hip.so (make -C {csrc}): newer sources {stale}"


def test_weight_reload_reaches_blocks_inside_module_lists(pkg):
    """Packed device weights are a cache of the nn.Parameters.  A reload through
    a container (blocks live in nn.ModuleList) must drop every nested cache:
    otherwise forward keeps computing with the old weights."""
    g = torch.Generator().manual_seed(5)
    stack = pkg.nn.PairformerStack(num_blocks=2)
    inner = stack.trunk_pairformer[1].triangle_multiplication_outgoing
    old = inner.packed()["w_out"].clone()
    assert inner._packed is not None
    new_state = {k: torch.randn(v.shape, generator=g) for k, v in stack.state_dict().items()}
    stack.load_state_dict(new_state)
    assert inner._packed is None
    key = "trunk_pairformer.1.triangle_multiplication_outgoing.output_projection.weight"
    assert torch.equal(inner.packed()["w_out"], new_state[key].to(torch.bfloat16))
    assert not torch.equal(inner.packed()["w_out"], old)
    # load_hip_params on the container packs every nested module as well
    stack.invalidate()
    assert all(m._packed is None for m in stack.modules() if isinstance(m, pkg.nn.base.HipModule))
    stack.load_hip_params()
    assert all(m._packed is not None for m in stack.modules() if isinstance(m, pkg.nn.base.HipModule))
    dt = pkg.nn.DiffusionTransformer(num_blocks=2, super_block_size=2, use_batch_infer=True)
    dt.load_hip_params()
    blk = dt.self_attention[1]
    assert blk._packed is not None
    dt.load_state_dict(dt.state_dict())
    assert blk._packed is None
