"""Pins of the diffusion-head oracle (oracle/af3_head_oracle.py) and of the
product's pure-PyTorch layout / schedule helpers (nn/atom_layout.py,
nn/diffusion_head.py), on the CPU.

The oracle's vectorised code is checked against brute-force loops over single
atoms and token pairs written independently of it, against closed forms
(schedule end points, zero output weights) and against invariants (a rigid
motion keeps distances, layout gathers are inverse to each other)."""

import math

import pytest
import torch

from oracle import af3_head_oracle as H
from oracle import af3_oracle as O

D = torch.float64


@pytest.fixture(scope="module")
def AL(pkg):
    return pkg.nn.atom_layout


def gen(seed):
    return torch.Generator().manual_seed(seed)


def tiny_batch(AL, n=8, seed=3, pad=1):
    return AL.synthetic_batch(n, gen(seed), n_padding_tokens=pad, chain_len=3)


# ------------------------------------------------------------------ layout

def test_convert_is_a_masked_gather(AL):
    g = gen(0)
    arr = torch.randn(2, 4, 6, 5, generator=g, dtype=D)          # layout axes (1, 2): 24 slots
    idx = torch.randint(0, 24, (3, 7), generator=g)
    msk = torch.rand(3, 7, generator=g) > 0.3
    gi = AL.GatherInfo(idx, msk, (4, 6))
    for conv in (H.convert, AL.convert):
        out = conv(gi, arr, (-3, -2))
        assert out.shape == (2, 3, 7, 5)
        for b in range(2):
            for i in range(3):
                for j in range(7):
                    r, c = divmod(int(idx[i, j]), 6)
                    want = arr[b, r, c] if msk[i, j] else torch.zeros(5, dtype=D)
                    assert torch.equal(out[b, i, j], want)
        with pytest.raises(ValueError):
            conv(gi, arr[:, :3], (-3, -2))                        # 18 slots for a 24-slot gather


def test_layout_gathers_are_consistent(AL):
    b = tiny_batch(AL, n=12, pad=2)
    aca, am = b.atom_cross_att, b.predicted_structure_info.atom_mask.bool()
    n, a = am.shape
    t2q, q2t, q2k = aca.token_atoms_to_queries, aca.queries_to_token_atoms, aca.queries_to_keys
    # every atom that is present sits in exactly one query slot, in token order
    real = t2q.gather_idxs[t2q.gather_mask]
    assert torch.equal(real, torch.arange(n * a).reshape(n, a)[am])
    assert int(t2q.gather_mask.sum()) == int(am.sum())
    # token-atoms -> queries -> token-atoms is the identity on the atoms that are present
    x = torch.randn(n, a, 3, generator=gen(1), dtype=D) * am[..., None]
    assert torch.equal(H.convert(q2t, H.convert(t2q, x, (-3, -2)), (-3, -2)), x)
    # tokens_to_queries is the token of each query atom
    assert torch.equal(aca.tokens_to_queries.gather_idxs[t2q.gather_mask], (real // a))
    # every subset's own 32 queries lie inside its window of 128 keys
    s = q2k.gather_idxs.shape[0]
    for i in range(s):
        win = set(q2k.gather_idxs[i].tolist())
        assert len(win) == 128 and set(range(32 * i, 32 * i + 32)) <= win
    assert torch.equal(q2k.gather_mask, t2q.gather_mask.reshape(-1)[q2k.gather_idxs])
    assert torch.equal(aca.tokens_to_keys.gather_idxs, aca.tokens_to_queries.gather_idxs.reshape(-1)[q2k.gather_idxs])


def test_mask_mean_brute_force():
    g = gen(2)
    v = torch.randn(2, 5, 4, 3, generator=g, dtype=D)
    m = (torch.rand(1, 5, 4, 1, generator=g) > 0.4).to(D)
    m[0, 2] = 0                                                   # a token without atoms
    got = H.mask_mean(m, v, dim=-2)
    for b in range(2):
        for t in range(5):
            cnt = float(m[0, t, :, 0].sum())
            for c in range(3):
                tot = sum(float(v[b, t, a, c]) for a in range(4) if m[0, t, a, 0] > 0)
                assert abs(float(got[b, t, c]) - (tot / cnt if cnt else 0.0)) < 1e-12


# ------------------------------------------------------------------ features

def rel_encoding_loop(tf, r=32, c=2):
    n = tf.asym_id.shape[0]
    out = torch.zeros(n, n, 2 * (2 * r + 2) + 1 + 2 * c + 2)
    for i in range(n):
        for j in range(n):
            same_chain = int(tf.asym_id[i]) == int(tf.asym_id[j])
            d = min(max(int(tf.residue_index[i]) - int(tf.residue_index[j]) + r, 0), 2 * r) if same_chain else 2 * r + 1
            out[i, j, d] = 1
            same_res = same_chain and int(tf.residue_index[i]) == int(tf.residue_index[j])
            d = min(max(int(tf.token_index[i]) - int(tf.token_index[j]) + r, 0), 2 * r) if same_res else 2 * r + 1
            out[i, j, 2 * r + 2 + d] = 1
            same_ent = int(tf.entity_id[i]) == int(tf.entity_id[j])
            out[i, j, 2 * (2 * r + 2)] = float(same_ent)
            d = min(max(int(tf.sym_id[i]) - int(tf.sym_id[j]) + c, 0), 2 * c) if same_ent else 2 * c + 1
            out[i, j, 2 * (2 * r + 2) + 1 + d] = 1
    return out


def test_relative_encoding_brute_force(pkg, AL):
    # chains of 5 tokens, several tokens per residue, copies of one entity, and a long chain for the clipping
    n = 90
    idx = torch.arange(n)
    tf = AL.TokenFeatures(mask=torch.ones(n), token_index=idx, residue_index=torch.where(idx < 80, idx // 2, idx),
                          asym_id=torch.where(idx < 80, 1, 2 + (idx - 80) // 5),
                          entity_id=torch.where(idx < 80, 1, 2), sym_id=torch.where(idx < 80, 1, 1 + (idx - 80) // 5))
    want = rel_encoding_loop(tf)
    assert want.shape[-1] == 139
    assert torch.equal(H.create_relative_encoding(tf).float(), want)
    prod = pkg.nn.diffusion_head.create_relative_encoding(tf)
    assert torch.equal(prod.float(), want)
    assert torch.equal(want.sum(-1) - want[..., 132], torch.full((n, n), 3.0))   # three one-hot groups


def test_fourier_and_noise_schedule_closed_forms(pkg):
    g = gen(4)
    x, w, b = torch.randn(5, generator=g, dtype=D), torch.randn(7, generator=g, dtype=D), torch.rand(7, generator=g, dtype=D)
    got = H.fourier_embeddings(x, w, b)
    for i in range(5):
        for j in range(7):
            assert abs(float(got[i, j]) - math.cos(2 * math.pi * (float(x[i]) * float(w[j]) + float(b[j])))) < 1e-12
    t = torch.linspace(0, 1, 11, dtype=D)
    s = H.noise_schedule(t)
    assert abs(float(s[0]) - 16.0 * 160.0) < 1e-9 and abs(float(s[-1]) - 16.0 * 0.0004) < 1e-12
    assert bool((s[1:] < s[:-1]).all())
    mid = 16.0 * (0.5 * 160.0 ** (1 / 7) + 0.5 * 0.0004 ** (1 / 7)) ** 7
    assert abs(float(s[5]) - mid) < 1e-9
    assert torch.allclose(pkg.nn.diffusion_head.noise_schedule(t), s)
    # sampler schedule: t_hat = previous level * (1 + 0.8 [level > 1]); noise_scale^2 = 1.003^2 (t_hat^2 - prev^2)
    lv, th, ns = H.sampler_schedule(10)
    for i in range(10):
        gamma = 0.8 if float(lv[i + 1]) > 1.0 else 0.0
        assert abs(float(th[i]) - float(lv[i]) * (1 + gamma)) < 1e-9
        assert abs(float(ns[i]) - 1.003 * math.sqrt(float(th[i]) ** 2 - float(lv[i]) ** 2)) < 1e-9
    sm = pkg.nn.DiffusionSampler(None, diffusion_steps=10)
    for a, b2 in zip(sm.schedule("cpu"), (lv, th, ns)):
        assert torch.allclose(a.double(), b2, rtol=1e-5)


def test_random_augmentation_is_a_rigid_motion(pkg):
    g = gen(5)
    pos = torch.randn(2, 6, 4, 3, generator=g, dtype=D) * 5
    mask = torch.rand(6, 4, generator=g) > 0.3
    rot = pkg.nn.diffusion_head.random_rotation(g, "cpu", D)
    assert torch.allclose(rot @ rot.T, torch.eye(3, dtype=D), atol=1e-12) and abs(float(torch.det(rot)) - 1) < 1e-12
    trans = torch.randn(3, generator=g, dtype=D)
    for fn in (H.random_augmentation, pkg.nn.diffusion_head.random_augmentation):
        out = fn(pos, mask[None], rot, trans)
        assert torch.equal(out[:, ~mask], torch.zeros_like(out[:, ~mask]))
        for s in range(2):
            a, b = pos[s][mask], out[s][mask]
            assert torch.allclose(torch.cdist(a, a), torch.cdist(b, b), atol=1e-10)
            assert torch.allclose(b.mean(0), trans, atol=1e-10)   # the masked mean moves to the translation


# ------------------------------------------------------------------ encoder / decoder by single atoms

def head_case(AL, n=8, blocks=1, seed=7, samples=2):
    g = gen(seed)
    b = tiny_batch(AL, n=n, seed=seed)
    p = H.make_diffusion_head_params(g, num_blocks=blocks, std=0.05, dtype=D)
    emb = {"single": torch.randn(n, 384, generator=g, dtype=D), "pair": torch.randn(n, n, 128, generator=g, dtype=D),
           "target_feat": torch.randn(n, 447, generator=g, dtype=D)}
    pos = torch.randn(samples, n, 24, 3, generator=g, dtype=D)
    return g, b, p, emb, pos


def test_encoder_conditioning_by_single_atoms(AL):
    g, b, p, emb, pos = head_case(AL)
    pe = O._sub(p, "atom_cross_att_encoder")
    n, a = 8, 24
    trunk_pair = torch.randn(n, n, 128, generator=g, dtype=D)
    enc = H.atom_cross_att_encoder(b, pos, emb["single"], trunk_pair, pe, True)
    rs, aca = b.ref_structure, b.atom_cross_att
    am = b.predicted_structure_info.atom_mask.bool()
    flat = [(t, s) for t in range(n) for s in range(a) if am[t, s]]      # flat atom -> (token, slot)
    lnw = pe["lnorm_trunk_single_cond.weight"]

    def ln(x, w):
        mu = x.mean()
        return (x - mu) / torch.sqrt(((x - mu) ** 2).mean() + 1e-5) * w

    def cond_of(f):
        t, s = flat[f]
        v = pe["embed_ref_pos.weight"] @ rs.positions[t, s].double() + pe["embed_ref_mask.weight"][:, 0] * 1.0
        v = v + pe["embed_ref_element.weight"][:, int(rs.element[t, s])]
        v = v + pe["embed_ref_charge.weight"][:, 0] * math.asinh(float(rs.charge[t, s]))
        for j in range(4):
            v = v + pe["embed_ref_atom_name.weight"][:, 64 * j + int(rs.atom_name_chars[t, s, j])]
        return v + pe["embed_trunk_single_cond.weight"] @ ln(emb["single"][t], lnw)

    n_real = len(flat)
    q2k = aca.queries_to_keys
    uid_flat = rs.ref_space_uid.reshape(-1)
    tp_w, tp_ln = pe["embed_trunk_pair_cond.weight"], pe["lnorm_trunk_pair_cond.weight"]
    checked = 0
    for (s, q, k) in [(0, 0, 0), (0, 5, 77), (1, 31, 3), (2, 7, 120), (3, 2, 64), (n_real // 32, 1, 127)]:
        f = 32 * s + q
        kf = int(q2k.gather_idxs[s, k])
        if f >= n_real:
            continue
        cq = cond_of(f)
        assert torch.allclose(enc.queries_single_cond[s, q], cq, atol=1e-10)
        k_real = kf < n_real
        ck = cond_of(kf) if k_real else torch.zeros(128, dtype=D)
        assert torch.allclose(enc.keys_single_cond[s, k], ck, atol=1e-10)
        assert bool(enc.keys_mask[s, k]) == k_real
        want = pe["single_to_pair_cond_row_1.weight"] @ torch.relu(cq) + pe["single_to_pair_cond_col_1.weight"] @ torch.relu(ck)
        (tq, sq_) = flat[f]
        pk = torch.zeros(3, dtype=D)
        if k_real:
            (tk, sk) = flat[kf]
            want = want + tp_w @ ln(trunk_pair[tq, tk], tp_ln)
            pk = rs.positions[tk, sk].double()
        # the key's frame id is read from the token-atom table at the QUERY-layout index (as the reference does)
        k_uid = int(uid_flat[kf]) if k_real else 0
        valid = 1.0 if int(rs.ref_space_uid[tq, sq_]) == k_uid else 0.0
        off = rs.positions[tq, sq_].double() - pk
        want = want + valid * (pe["embed_pair_offsets_1.weight"] @ off)
        want = want + valid * pe["embed_pair_distances_1.weight"][:, 0] / (1 + float(off @ off))
        want = want + valid * pe["embed_pair_offsets_valid.weight"][:, 0]
        h = pe["pair_mlp_2.weight"] @ torch.relu(pe["pair_mlp_1.weight"] @ torch.relu(want))
        want = want + pe["pair_mlp_3.weight"] @ torch.relu(h)
        assert torch.allclose(enc.pair_cond[s, q, k], want, atol=1e-9), (s, q, k)
        checked += 1
    assert checked >= 5
    # aggregation to tokens: mean over a token's atoms of relu(project(atom activation))
    w = pe["project_atom_features_for_aggr.weight"]
    for t in (0, 3, n - 2):
        atoms = [f for f, (tt, _) in enumerate(flat) if tt == t]
        for smp in range(2):
            want = sum(torch.relu(w @ enc.skip_connection[smp].reshape(-1, 128)[f]) for f in atoms) / len(atoms)
            assert torch.allclose(enc.token_act[smp, t], want, atol=1e-10)
    assert torch.equal(enc.token_act[:, n - 1], torch.zeros_like(enc.token_act[:, n - 1]))   # padding token


def test_decoder_broadcast_and_scatter_by_single_atoms(AL):
    g, b, p, emb, pos = head_case(AL)
    pe, pd = O._sub(p, "atom_cross_att_encoder"), O._sub(p, "atom_cross_att_decoder")
    n, a = 8, 24
    trunk_pair = torch.randn(n, n, 128, generator=g, dtype=D)
    enc = H.atom_cross_att_encoder(b, pos, emb["single"], trunk_pair, pe, True)
    tok = torch.randn(2, n, 768, generator=g, dtype=D)
    upd = H.atom_cross_att_decoder(b, tok, enc, pd, True)
    am = b.predicted_structure_info.atom_mask.bool()
    flat = [(t, s) for t in range(n) for s in range(a) if am[t, s]]
    # rebuild the decoder input atom by atom, run the (separately pinned) transformer, scatter atom by atom
    q_in = torch.zeros(2, len(flat) // 32 * 32 + 32 * ((len(flat) % 32) > 0) + 0, 128, dtype=D)
    q_in = torch.zeros(2, n * a, 128, dtype=D)
    for f, (t, _) in enumerate(flat):
        for smp in range(2):
            q_in[smp, f] = pd["project_token_features_for_broadcast.weight"] @ tok[smp, t] \
                + enc.skip_connection[smp].reshape(-1, 128)[f]
    q2k = b.atom_cross_att.queries_to_keys
    q_out = O.cross_att_transformer(q_in.reshape(2, -1, 32, 128), enc.queries_mask, q2k.gather_idxs, q2k.gather_mask,
                                    enc.keys_mask, enc.queries_single_cond, enc.keys_single_cond, enc.pair_cond,
                                    O._sub(pd, "atom_transformer_decoder")).reshape(2, -1, 128)
    lnw = pd["atom_features_layer_norm.weight"]
    want = torch.zeros(2, n, a, 3, dtype=D)
    for f, (t, s) in enumerate(flat):
        for smp in range(2):
            x = q_out[smp, f]
            x = (x - x.mean()) / torch.sqrt(x.var(unbiased=False) + 1e-5) * lnw
            want[smp, t, s] = pd["atom_features_to_position_update.weight"] @ x
    assert torch.allclose(upd, want, atol=1e-9)


def test_head_closed_form_with_zero_update_weights(AL):
    g, b, p, emb, pos = head_case(AL)
    p = dict(p)
    p["atom_cross_att_decoder.atom_features_to_position_update.weight"] = torch.zeros(3, 128, dtype=D)
    lv, th, ns = H.sampler_schedule(2)
    sc, pc = H.pre_conditioning(b, emb, th, True, p)
    am = b.predicted_structure_info.atom_mask.double()[None, ..., None]
    t = th[1]
    out = H.diffusion_head(pos, t, b, emb, sc[1], pc, p, True, 1)
    assert torch.allclose(out, pos * am * 256.0 / (float(t) ** 2 + 256.0), atol=1e-12)
    # two sampler steps with the denoiser reduced to skip * noisy: closed-form update per step
    rots = torch.stack([torch.eye(3, dtype=D)] * 2)
    transs = torch.zeros(2, 3, dtype=D)
    got = H.sample_diffusion(b, emb, p, pos, rots, transs, steps=2, num_blocks=1)
    x = pos * lv[0]
    for i in range(2):
        m = am
        centre = (x * m).sum(dim=(1, 2), keepdim=True) / m.sum()
        x = (x - centre) * m
        noisy = x + ns[i]
        den = noisy * m * 256.0 / (float(th[i]) ** 2 + 256.0)
        x = noisy + 1.5 * (lv[i + 1] - th[i]) * (noisy - den) / th[i]
    assert torch.allclose(got, x, atol=1e-9)


def test_pre_conditioning_rows_are_independent_of_the_other_noise_levels(AL):
    """single_cond[i] depends on noise level i only, pair_cond on none: the
    head may be fed one row at a time (d_alphafold3.py:392-398)."""
    g, b, p, emb, pos = head_case(AL)
    lv, th, ns = H.sampler_schedule(4)
    sc, pc = H.pre_conditioning(b, emb, th, True, p)
    sc1, pc1 = H.pre_conditioning(b, emb, th[2:3], True, p)
    assert torch.allclose(sc[2], sc1[0], atol=1e-12) and torch.allclose(pc, pc1, atol=1e-12)
    # use_conditioning = 0 removes the trunk embeddings but keeps the relative encoding and target features
    emb0 = dict(emb, single=torch.zeros_like(emb["single"]), pair=torch.zeros_like(emb["pair"]))
    a = H.pre_conditioning(b, emb, th, 0.0, p)
    z = H.pre_conditioning(b, emb0, th, 1.0, p)
    assert torch.allclose(a[0], z[0], atol=1e-12) and torch.allclose(a[1], z[1], atol=1e-12)
