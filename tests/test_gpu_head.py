"""Diffusion head on the GPU (HIP kernels through the C ABI) against the CPU
oracle in float64 (oracle/af3_head_oracle.py), at sizes the oracle finishes in
seconds, and size-independent properties at 768 tokens x 5 samples.

Tolerances: bf16 path rms error of the position UPDATE (denoised minus the
skip term) <= 1e-2 of its rms, max <= 8e-2; fp32 check mode 2e-4 / 2e-3."""

import pytest
import torch

from oracle import af3_head_oracle as H
from oracle import af3_oracle as O

pytestmark = pytest.mark.gpu
D = torch.float64


def dev():
    return torch.device("cuda:0")


def gen(seed):
    return torch.Generator().manual_seed(seed)


def compare(name, got, ref, rms_tol, max_tol):
    got, ref = got.double().cpu(), ref.double().cpu()
    scale = float((ref ** 2).mean().sqrt())
    rms = float(((got - ref) ** 2).mean().sqrt()) / scale
    mx = float((got - ref).abs().max()) / scale
    print(f"head {name}: rms {rms:.3e} max {mx:.3e} (rms of reference {scale:.3e})", flush=True)
    assert torch.isfinite(got).all() and scale > 0
    assert rms <= rms_tol and mx <= max_tol, (name, rms, mx)


def case(pkg, n, blocks, seed, samples=2, pad=1, std=0.05):
    g = gen(seed)
    batch = pkg.nn.atom_layout.synthetic_batch(n, g, n_padding_tokens=pad, chain_len=5)
    p = {k: O.round_bf16(v) for k, v in H.make_diffusion_head_params(g, num_blocks=blocks, std=std).items()}
    emb = {"single": O.round_bf16(torch.randn(n, 384, generator=g)),
           "pair": O.round_bf16(torch.randn(n, n, 128, generator=g)),
           "target_feat": O.round_bf16(torch.randn(n, 447, generator=g))}
    pos = torch.randn(samples, n, 24, 3, generator=g)
    head = pkg.nn.DiffusionHead(num_blocks=blocks)
    head.load_state_dict(p)
    head.to(dev())
    return g, batch, p, emb, pos, head


def on_gpu(emb):
    return {k: v.to(dev()) for k, v in emb.items()}


@pytest.mark.parametrize("n,blocks", [(8, 1), (20, 4)])
def test_pre_conditioning_and_head_against_oracle(gpu_pkg, n, blocks):
    g, batch, p, emb, pos, head = case(gpu_pkg, n, blocks, seed=21 + n)
    pd = O.cast_params(p, D)
    embd = {k: v.double() for k, v in emb.items()}
    levels, t_hat, _ = H.sampler_schedule(6)
    want_sc, want_pc = H.pre_conditioning(batch, embd, t_hat, True, pd)
    gb, ge = batch.to(dev()), on_gpu(emb)
    for mode, rms_tol, max_tol in (("check", 2e-4, 2e-3), ("bf16", 1e-2, 8e-2)):
        with gpu_pkg.nn.check_mode(mode == "check"):
            sc, pc = head.pre_conditioning(gb, ge, t_hat.float().to(dev()), True)
            compare(f"single_cond {mode}", sc, want_sc, rms_tol, max_tol)
            compare(f"pair_cond {mode}", pc, want_pc, rms_tol, max_tol)
            for step in (0, 3, 5):          # high, middle and low noise
                t = t_hat[step]
                noisy = pos.double() * float(t)
                want = H.diffusion_head(noisy, t, batch, embd, want_sc[step], want_pc, pd, True, blocks)
                got = head(noisy.float().to(dev()), t.float().to(dev()), gb, ge,
                           want_sc[step].float().to(dev()), want_pc.float().to(dev()))
                am = batch.predicted_structure_info.atom_mask.double()[None, ..., None]
                skip = 256.0 / (float(t) ** 2 + 256.0) * noisy * am
                compare(f"update, step {step}, {mode}", got.double().cpu() - skip, want - skip, rms_tol, max_tol)


@pytest.mark.parametrize("n,in_dtype", [(150, torch.float32), (96, torch.bfloat16)])
def test_pair_conditioning_first_layer_kernel(gpu_pkg, n, in_dtype):
    """ops.pair_cond_init against LayerNorm + projection of the explicit [pair | relative encoding] tensor
    in float64, on token features that reach every branch of the encoding: several chains, residues of
    several tokens (same residue, different token index), offsets beyond the clipping range, chain copies
    of one entity and chains of different entities."""
    print(f"test_pair_conditioning_first_layer_kernel n={n} {in_dtype}", flush=True)
    from types import SimpleNamespace
    g = gen(300 + n)
    ri = lambda lo, hi: torch.randint(lo, hi, (n,), generator=g)
    tf = SimpleNamespace(asym_id=ri(1, 4), residue_index=ri(0, 90) // ri(1, 3).clamp(max=2), token_index=ri(0, 80),
                         entity_id=ri(1, 3), sym_id=ri(1, 7))
    tf.residue_index[: n // 3] = tf.residue_index[0]      # a long residue: many tokens share it
    tf.asym_id[: n // 3] = tf.asym_id[0]
    pair = O.round_bf16(torch.randn(n, n, 128, generator=g) * 2 + 0.5)
    ln_w = 1 + 0.2 * torch.randn(267, generator=g)
    w = O.round_bf16(torch.randn(128, 267, generator=g) * 0.1)
    scale = 0.75
    f2d = torch.cat([scale * pair.double(), H.create_relative_encoding(tf).double()], dim=-1)
    want = torch.nn.functional.layer_norm(f2d, (267,), ln_w.double(), None, 1e-5) @ w.double().T
    ids = tuple(getattr(tf, k).to(torch.int32).to(dev()) for k in ("asym_id", "residue_index", "token_index", "entity_id", "sym_id"))
    g_hot = (w[:, 128:].float() * ln_w[128:]).t().contiguous()
    got = gpu_pkg.ops.pair_cond_init(pair.to(in_dtype).to(dev()), ids, ln_w[:128].contiguous().to(dev()),
                                     w[:, :128].contiguous().bfloat16().to(dev()), g_hot.to(dev()), g_hot.sum(0).to(dev()),
                                     in_scale=scale)
    compare("pair conditioning, first layer", got, want, 3.5e-3, 2e-2)
    # pair channels switched off: what is left is the one-hot share (fp32 table rows) and the pair channels'
    # LayerNorm shift; a wrong table row would show at the size of the output itself
    f2d0 = torch.cat([0 * pair.double(), H.create_relative_encoding(tf).double()], dim=-1)
    want0 = torch.nn.functional.layer_norm(f2d0, (267,), ln_w.double(), None, 1e-5) @ w.double().T
    got0 = gpu_pkg.ops.pair_cond_init(pair.to(in_dtype).to(dev()), ids, ln_w[:128].contiguous().to(dev()),
                                      w[:, :128].contiguous().bfloat16().to(dev()), g_hot.to(dev()), g_hot.sum(0).to(dev()),
                                      in_scale=0.0)
    compare("pair conditioning, one-hot share alone", got0, want0, 3e-4, 1e-3)


@pytest.mark.parametrize("with_tp", [True, False])
def test_atom_pair_conditioning_kernel(gpu_pkg, with_tp):
    """ops.atom_pair_cond against the same sum of terms and three-layer MLP written out in float64."""
    print(f"test_atom_pair_conditioning_kernel with_tp={with_tp}", flush=True)
    g = gen(512)
    S, Q, K, n_tok = 5, 32, 128, 11
    r = lambda *shape: torch.randn(*shape, generator=g)
    row, col, tp = r(S, Q, 16), r(S, K, 16), r(n_tok, n_tok, 16)
    tq = torch.randint(-1, n_tok, (S, Q), generator=g)
    tk = torch.randint(-1, n_tok, (S, K), generator=g)
    q_pos, k_pos = r(S, Q, 3) * 3, r(S, K, 3) * 3
    q_uid, k_uid = torch.randint(0, 4, (S, Q), generator=g), torch.randint(0, 4, (S, K), generator=g)
    w_off, w_dist, w_valid = r(16, 3), r(16, 1), r(16, 1)
    w1, w2, w3 = r(16, 16) * 0.4, r(16, 16) * 0.4, r(16, 16) * 0.4
    d = lambda t: t.double()
    a = d(row)[:, :, None, :] + d(col)[:, None, :, :]
    if with_tp:
        live = ((tq >= 0)[:, :, None] & (tk >= 0)[:, None, :])[..., None].double()
        a = a + d(tp)[tq.clamp(min=0)[:, :, None], tk.clamp(min=0)[:, None, :]] * live
    valid = (q_uid[:, :, None] == k_uid[:, None, :]).double()[..., None]
    off = d(q_pos)[:, :, None, :] - d(k_pos)[:, None, :, :]
    a = a + (off @ d(w_off).T + (1.0 / (1 + (off * off).sum(-1, keepdim=True))) @ d(w_dist).T + d(w_valid)[:, 0]) * valid
    h = torch.relu(a) @ d(w1).T
    h = torch.relu(h) @ d(w2).T
    want = a + torch.relu(h) @ d(w3).T
    t = lambda x: x.to(dev())
    i32 = lambda x: x.to(torch.int32).to(dev())
    got = gpu_pkg.ops.atom_pair_cond(t(row), t(col), t(tp) if with_tp else None, i32(tq) if with_tp else None,
                                     i32(tk) if with_tp else None, t(q_pos), t(k_pos), i32(q_uid), i32(k_uid),
                                     t(w_off), t(w_dist), t(w_valid), t(w1), t(w2), t(w3))
    compare("atom pair conditioning", got, want, 2e-6, 2e-5)


def test_atom_pair_logits_kernel(gpu_pkg):
    """ops.atom_pair_logits against LayerNorm + projection + the block / head split in float64."""
    print("test_atom_pair_logits_kernel", flush=True)
    g = gen(411)
    S, Q, K, blocks, heads = 7, 32, 128, 3, 4
    x = torch.randn(S, Q, K, 16, generator=g) * 3 + 1
    ln_w = 1 + 0.3 * torch.randn(16, generator=g)
    w = torch.randn(blocks * heads, 16, generator=g)
    want = torch.nn.functional.layer_norm(x.double(), (16,), ln_w.double(), None, 1e-5) @ w.double().T
    want = want.reshape(S, Q, K, blocks, heads).permute(3, 0, 4, 1, 2)
    got = gpu_pkg.ops.atom_pair_logits(x.to(dev()), ln_w.to(dev()), w.to(dev()), blocks, heads)
    assert tuple(got.shape) == (blocks, S, heads, Q, K)
    compare("atom pair logits", got, want, 2e-6, 2e-5)


def test_state_reuse_is_exact_and_samples_are_independent(gpu_pkg):
    g, batch, p, emb, pos, head = case(gpu_pkg, 16, 4, seed=31, samples=3)
    gb, ge = batch.to(dev()), on_gpu(emb)
    levels, t_hat, _ = H.sampler_schedule(4)
    sc, pc = head.pre_conditioning(gb, ge, t_hat.float().to(dev()), True)
    noisy = (pos * float(t_hat[2])).to(dev())
    state = head.prepare(gb, ge, pc)
    a = head(noisy, t_hat[2].float().to(dev()), gb, ge, sc[2], pc, state=state)
    b = head(noisy, t_hat[2].float().to(dev()), gb, ge, sc[2], pc)                  # conditioning recomputed
    c = head(noisy, t_hat[2].float().to(dev()), gb, ge, sc[2], pc, state=state)    # the state is not consumed
    assert torch.equal(a, b) and torch.equal(a, c)
    # a sample's result does not depend on which other samples share the batch
    one = head(noisy[1:2].contiguous(), t_hat[2].float().to(dev()), gb, ge, sc[2], pc, state=state)
    assert torch.equal(one[0], a[1])


def test_sampler_against_oracle(gpu_pkg):
    n, blocks, steps, samples = 12, 2, 4, 2
    g, batch, p, emb, pos, head = case(gpu_pkg, n, blocks, seed=41, samples=samples)
    pd = O.cast_params(p, D)
    embd = {k: v.double() for k, v in emb.items()}
    rots = torch.stack([gpu_pkg.nn.diffusion_head.random_rotation(g, "cpu", D) for _ in range(steps)])
    transs = torch.randn(steps, 3, generator=g, dtype=D)
    want = H.sample_diffusion(batch, embd, pd, pos.double(), rots, transs, steps, num_blocks=blocks)
    gb, ge = batch.to(dev()), on_gpu(emb)
    sampler = gpu_pkg.nn.DiffusionSampler(head, num_samples=samples, diffusion_steps=steps)
    for mode, rms_tol, max_tol in (("check", 2e-4, 2e-3), ("bf16", 1e-2, 8e-2)):
        with gpu_pkg.nn.check_mode(mode == "check"):
            out = sampler(gb, ge, positions=pos.to(dev()), rotations=rots.float().to(dev()),
                          translations=transs.float().to(dev()))
        assert torch.equal(out["mask"].cpu(), batch.predicted_structure_info.atom_mask)
        compare(f"sampled positions after {steps} steps, {mode}", out["atom_positions"], want, rms_tol, max_tol)
    # gaussian noise handed in: the oracle takes the same draws
    noises = torch.randn(steps, samples, n, 24, 3, generator=g, dtype=D)
    want = H.sample_diffusion(batch, embd, pd, pos.double(), rots, transs, steps, num_blocks=blocks, noises=noises)
    out = sampler(gb, ge, positions=pos.to(dev()), rotations=rots.float().to(dev()),
                  translations=transs.float().to(dev()), noises=noises.float().to(dev()))
    compare("sampled positions, gaussian noise", out["atom_positions"], want, 1e-2, 8e-2)


def test_full_size_head_properties(gpu_pkg):
    """768 tokens x 5 samples x 24 blocks: equal samples stay equal; a sample
    evaluated alone gives the same result as inside the batch; padding atoms
    stay at zero; one evaluation against the fp32 check mode."""
    n, samples = 768, 5
    g, batch, p, emb, pos, head = case(gpu_pkg, n, 24, seed=51, samples=samples, pad=40, std=0.02)
    gb, ge = batch.to(dev()), on_gpu(emb)
    levels, t_hat, _ = H.sampler_schedule(200)
    t = t_hat[120:121].float().to(dev())
    sc, pc = head.pre_conditioning(gb, ge, t, True)
    state = head.prepare(gb, ge, pc)
    am = gb.predicted_structure_info.atom_mask.bool()
    noisy = (pos * float(t)).to(dev())
    noisy[3] = noisy[0]
    out = head(noisy, t[0], gb, ge, sc[0], pc, state=state)
    assert torch.isfinite(out).all()
    assert torch.equal(out[3], out[0])
    assert torch.equal(out[:, ~am], torch.zeros_like(out[:, ~am]))
    one = head(noisy[2:3].contiguous(), t[0], gb, ge, sc[0], pc, state=state)
    assert torch.equal(one[0], out[2])
    with gpu_pkg.nn.check_mode():
        sc32, pc32 = head.pre_conditioning(gb, ge, t, True)
        ref = head(noisy[:1].contiguous(), t[0], gb, ge, sc32[0], pc32)
    # caps at 1.25 x the measured figures (rms / max over the rms of the check mode's result: conditioning
    # 1.8e-3 / 1.0e-2, update after 24 + 6 blocks of bf16 intermediates 8.9e-3 / 5.5e-2)
    compare("single_cond, bf16 vs fp32 check", sc, sc32, 2.5e-3, 1.3e-2)
    compare("pair_cond, bf16 vs fp32 check", pc, pc32, 2.5e-3, 1.3e-2)
    skip = 256.0 / (float(t) ** 2 + 256.0) * noisy[:1] * am[None, ..., None]
    compare("update, bf16 vs fp32 check", out[:1] - skip, ref - skip, 1.2e-2, 7e-2)


def test_per_atom_key_path_matches_the_gathered_key_tensor_path(gpu_pkg):
    """The atom transformer with keys looked up inside the attention kernel
    (K / V projected once per atom) against the same transformer fed the
    gathered key tensors, which is the reference's formulation."""
    g = gen(61)
    batch = gpu_pkg.nn.atom_layout.synthetic_batch(20, g, n_padding_tokens=3)
    q2k = batch.atom_cross_att.queries_to_keys.to(dev())
    s = q2k.gather_idxs.shape[0]
    p = {k: O.round_bf16(v) for k, v in O.make_cross_att_transformer_params(g, std=0.05).items()}
    mod = gpu_pkg.nn.DiffusionCrossAttTransformer()
    mod.load_state_dict(p)
    mod.to(dev())
    rb = O.round_bf16
    qm = batch.atom_cross_att.token_atoms_to_queries.gather_mask.to(dev())
    act = (rb(torch.randn(3, s, 32, 128, generator=g)).to(dev()) * qm[None, ..., None]).bfloat16()
    cq = rb(torch.randn(s, 32, 128, generator=g)).to(dev()) * qm[..., None]
    pc = rb(torch.randn(s, 32, 128, 16, generator=g)).to(dev())
    ck = gpu_pkg.nn.atom_layout.convert(q2k, cq, (-3, -2)).contiguous()
    km = gpu_pkg.nn.atom_layout.convert(q2k, qm, (-2, -1))
    plain = mod(act.clone(), qm, q2k, km, cq, ck, pc)
    cond = mod.conditioning(cq, ck, pc, keys_are_query_atoms=q2k)
    fast = mod(act.clone(), qm, q2k, km, cq, ck, pc, cond=cond)
    live = qm[None, ..., None]
    compare("per-atom keys vs gathered keys", ((fast - act) * live).float(), ((plain - act) * live).float(), 2e-3, 3e-2)


def test_encoder_without_positions_and_trunk_conditioning(gpu_pkg):
    """The encoder as the trunk's input embedder uses it (d_alphafold3.py:303-308:
    no atom positions, no trunk conditioning, 384 token channels, no sample axis)."""
    g = gen(71)
    n = 12
    batch = gpu_pkg.nn.atom_layout.synthetic_batch(n, g, n_padding_tokens=2, chain_len=5)
    p = {k: O.round_bf16(v) for k, v in H.make_encoder_params(g, 384, False, False, False, std=0.05).items()}
    want = H.atom_cross_att_encoder(batch, None, None, None, O.cast_params(p, D), batched=False)
    enc = gpu_pkg.nn.AtomCrossAttEncoder()
    enc.load_state_dict(p)
    enc.to(dev())
    gb = batch.to(dev())
    for mode, rms_tol, max_tol in (("check", 2e-4, 2e-3), ("bf16", 1e-2, 8e-2)):
        with gpu_pkg.nn.check_mode(mode == "check"):
            got = enc(batch=gb, token_atoms_act=None, trunk_single_cond=None, trunk_pair_cond=None)
        assert got.token_act.shape == (n, 384)
        compare(f"token_act {mode}", got.token_act, want.token_act, rms_tol, max_tol)
        compare(f"pair_cond {mode}", got.pair_cond, want.pair_cond, 1e-5, 1e-4)
        live = want.queries_mask[..., None]
        compare(f"skip connection {mode}", got.skip_connection.float().cpu() * live, want.skip_connection * live,
                rms_tol, max_tol)


@pytest.mark.parametrize("b,n_src,t,a,c", [(1, 40, 7, 5, 16), (3, 500, 61, 24, 768), (2, 96, 10, 32, 128)])
def test_gathered_relu_mean(gpu_pkg, b, n_src, t, a, c):
    """Atoms -> tokens aggregation (conversion to the token-atom layout, ReLU,
    masked mean) in one kernel against the same steps in torch."""
    print(f"test_gathered_relu_mean b={b} n_src={n_src} t={t} a={a} c={c}", flush=True)
    g = torch.Generator().manual_seed(t)
    src = torch.randn(b, n_src, c, generator=g).bfloat16()
    idx = torch.randint(0, n_src, (t, a), generator=g)
    present = torch.rand(t, a, generator=g) > 0.3
    present[0] = False                       # a token without atoms: zero sum over the clamped count
    present[1] = True
    count = torch.clamp(present.float().sum(-1), min=1e-10)
    rows = torch.where(present, idx, -1).to(torch.int32)
    dev = torch.device("cuda:0")
    got = gpu_pkg.ops.gathered_relu_mean(src.to(dev), rows.to(dev), count.to(dev)).cpu()
    gathered = src.float()[:, idx.reshape(-1)].reshape(b, t, a, c) * present[None, :, :, None]
    want = torch.relu(gathered).double().sum(-2) / count.double()[None, :, None]
    assert got.shape == (b, t, c)
    assert float((got.double() - want).abs().max()) <= 1e-6 * float(want.abs().max()) + 1e-30
    assert torch.all(got[:, 0] == 0)
    with pytest.raises(ValueError):
        gpu_pkg.ops.gathered_relu_mean(src.to(dev), (rows + n_src).to(dev), count.to(dev))


@pytest.mark.parametrize("b,n_slots,q,c,dt", [(1, 30, 64, 16, torch.float32), (5, 720, 736, 128, torch.bfloat16)])
def test_atom_position_features(gpu_pkg, b, n_slots, q, c, dt):
    """Position embedding at the head of the atom encoder (layout conversion, 3 -> c
    projection, query mask, + conditioning) in one kernel against the same steps in torch."""
    print(f"test_atom_position_features b={b} n_slots={n_slots} q={q} c={c} {dt}", flush=True)
    g = torch.Generator().manual_seed(q)
    pos = torch.randn(b, n_slots, 3, generator=g)
    rows = torch.randint(0, n_slots, (q,), generator=g)
    live = torch.rand(q, generator=g) > 0.2
    w, cond = torch.randn(c, 3, generator=g), torch.randn(q, c, generator=g)
    dev = torch.device("cuda:0")
    rows32 = torch.where(live, rows, -1).to(torch.int32)
    got = gpu_pkg.ops.atom_position_features(pos.to(dev), rows32.to(dev), w.to(dev), cond.to(dev), out_dtype=dt).cpu()
    want = (pos[:, rows].double() * live[None, :, None]) @ w.double().T + cond.double()
    assert got.shape == (b, q, c) and got.dtype == dt
    tol = 2.0 ** -8 if dt == torch.bfloat16 else 1e-6
    assert float((got.double() - want).abs().max()) <= tol * float(want.abs().max())
    assert torch.equal(got[:, ~live].float(), cond[~live].to(dt).float()[None].expand(b, -1, -1))


def test_head_without_batch_inference_matches_the_batched_head(gpu_pkg):
    """use_batch_infer=False (one sample, positions [N, A, 3], as the reference's
    unbatched modules take them) runs the same kernels on a batch of one: the
    update equals the batched head's on the same sample."""
    g, batch, p, emb, pos, head = case(gpu_pkg, 20, 2, seed=77, samples=2)
    single = gpu_pkg.nn.DiffusionHead(False, num_blocks=2)
    single.load_state_dict(p)
    single.to(dev())
    gb, ge = batch.to(dev()), on_gpu(emb)
    levels, t_hat, _ = H.sampler_schedule(4)
    t = t_hat[1].float().to(dev())
    sc, pc = head.pre_conditioning(gb, ge, t_hat.float().to(dev()), True)
    noisy = (pos * float(t_hat[1])).to(dev())
    want = head(noisy, t, gb, ge, sc[1], pc)
    for i in range(2):
        got = single(noisy[i], t, gb, ge, sc[1], pc)
        assert got.shape == want[i].shape
        err = float((got - want[i]).abs().max()) / float(want[i].abs().max())
        print(f"unbatched head, sample {i}: max difference {err:.3e}", flush=True)
        assert err <= 1e-6


def test_decoder_layout_kernels(gpu_pkg):
    """The two fused steps of the atom decoder against the same steps in torch:
    token rows gathered to the queries + skip connection (bit-identical), and
    LayerNorm -> position update -> token-atom layout."""
    print("test_decoder_layout_kernels", flush=True)
    g = torch.Generator().manual_seed(5)
    d = torch.device("cuda:0")
    b, n_tok, q, c = 3, 50, 416, 128
    src = torch.randn(b, n_tok, c, generator=g).bfloat16()
    add = torch.randn(b, q, c, generator=g).bfloat16()
    tok = torch.randint(0, n_tok, (q,), generator=g)
    live = torch.rand(q, generator=g) > 0.25
    rows = torch.where(live, tok, -1).to(torch.int32)
    got = gpu_pkg.ops.gather_rows_add(src.to(d), rows.to(d), add.to(d)).cpu()
    want = (src[:, tok] * live[None, :, None].to(torch.bfloat16)) + add
    assert torch.equal(got, want)
    # position update
    x = (torch.randn(b, q, c, generator=g) * 2 + 0.3).bfloat16()
    ln_w, w = torch.randn(c, generator=g), torch.randn(3, c, generator=g) * 0.1
    t_out = 77
    qi = torch.randint(0, q, (t_out,), generator=g)
    present = torch.rand(t_out, generator=g) > 0.3
    rows2 = torch.where(present, qi, -1).to(torch.int32)
    got = gpu_pkg.ops.position_update(x.to(d), rows2.to(d), ln_w.to(d), w.to(d)).cpu()
    y = torch.nn.functional.layer_norm(x.double(), (c,), ln_w.double(), None, 1e-5).float().bfloat16().double()
    want = (y @ w.double().T)[:, qi] * present[None, :, None]
    assert got.shape == (b, t_out, 3)
    err = float((got.double() - want).abs().max()) / float(want.abs().max())
    print(f"  position update: max difference {err:.3e} of the largest value", flush=True)
    assert err <= 2e-3        # a bf16 rounding of a normalised value may fall the other way
    assert torch.all(got[:, ~present] == 0)
