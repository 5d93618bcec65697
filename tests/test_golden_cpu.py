"""CPU checks of the committed fixtures: the configs[0] golden (made by tests/golden/make_golden.py) and the
vectors recorded from the reference's own code (tests/golden/make_reference_vectors.py)."""
import os

import numpy as np
import torch

from hashattention.synthetic import make_problem, named_workload, sha256_of
from oracle import c_oracle
from oracle import hashattn_oracle as orc

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _bits(a):
    return np.unpackbits(a.view(np.uint8))


def test_config0_inputs_are_reproducible_and_golden_holds():
    g = np.load(os.path.join(HERE, "config0.npz"))
    w = named_workload("config0")
    p = make_problem(w)
    assert sha256_of(p.q) == str(g["sha_q"]) and sha256_of(p.k) == str(g["sha_k"]) and sha256_of(p.v) == str(g["sha_v"])
    kcodes, qcodes = g["kcodes"], g["qcodes"]                       # [1,32,4096,1], [1,32,1,1] uint32
    # integer stages from the stored codes are exact on every machine
    idx, counts = c_oracle.select(kcodes, qcodes[:, :, 0], [4096], w.init_budget, w.recent_budget, w.heavy_budget, 1280)
    assert (counts == 1280).all() and np.array_equal(counts[0], g["n_selected"])
    mask = np.zeros((32, 4096), dtype=bool)
    for h in range(32):
        mask[h, idx[0, h]] = True
    assert np.array_equal(np.packbits(mask, axis=-1), g["mask"])
    # python formulation of the same selection
    ham = orc.hamming(torch.from_numpy(qcodes[:, :, 0].astype(np.int64)), torch.from_numpy(kcodes.astype(np.int64)))
    sel = orc.select_indices_np(ham[0].numpy(), 4096, w.init_budget, w.recent_budget, w.heavy_budget)
    assert np.array_equal(sel, idx[0])
    # attention over the golden index lists
    out = c_oracle.sparse_attend(p.q[:, :, 0], p.k, p.v, idx, counts, 1.0 / np.sqrt(128))
    assert np.abs(out[0] - g["out"]).max() < 2e-5
    # codes recomputed on this machine may differ from the stored ones only where a logit is ~0
    kl = orc.usa_logits(orc.repeat_kv(p.k, 4), p.usa.k)
    mine = orc.pack_codes(kl).numpy().astype(np.uint32)
    diff = mine ^ kcodes
    nflip = int(_bits(diff).sum())
    assert nflip <= int(g["near_zero_logits"][0])
    if nflip:
        bits = ((diff[..., None] >> np.arange(32, dtype=np.uint32)) & 1).astype(bool)[:, :, :, 0, :]
        assert (np.abs(kl.numpy())[bits] < 1e-4).all()


def _usa_heads(g, prefix="w", leaf=False):
    keys = [str(k) for k in g["state_keys"]]
    sd = {k: torch.from_numpy(g[f"{prefix}{i}"]).clone().requires_grad_(leaf) for i, k in enumerate(keys)}
    heads = {"k": [], "q": []}
    for side in ("k", "q"):
        h = 0
        while f"learning_to_hash_transformation_{side}.{h}.0.weight" in sd:
            layers = []
            for l in (0, 2, 4):
                pre = f"learning_to_hash_transformation_{side}.{h}.{l}"
                if pre + ".weight" in sd:
                    layers.append((sd[pre + ".weight"], sd[pre + ".bias"]))
            heads[side].append(layers)
            h += 1
    return heads


def test_oracle_matches_vectors_recorded_from_the_reference():
    """USA.forward(hard=True) and compute_mask_multi of the reference, as recorded from its own code."""
    g = np.load(os.path.join(HERE, "reference_vectors.npz"))
    heads = _usa_heads(g)
    assert len(heads["k"]) == 4 and len(heads["k"][0]) == 3
    K = torch.from_numpy(g["K"])
    Krep = orc.repeat_kv(K, 2)
    for name in ("q1", "q5"):
        Q = torch.from_numpy(g[f"{name}_Q"])
        span, ksign = orc.usa_forward_hard(Krep, Q, heads["k"], heads["q"])
        ref_span = torch.from_numpy(g[f"{name}_span"])
        assert torch.equal(span, ref_span)                     # integer-valued: exact
        assert np.array_equal(ksign.numpy().astype(np.int8), g[f"{name}_ksign"])
        # span = D - 2 * Hamming of the packed codes, wherever the reference's causal mask keeps it
        kc = orc.pack_codes(orc.usa_logits(Krep, heads["k"]))
        qc = orc.pack_codes(orc.usa_logits(Q, heads["q"]))
        for t in range(Q.shape[2]):
            ham = orc.hamming(qc[:, :, t], kc)
            keep = ref_span[:, :, t] > -1e30
            assert torch.equal((32 - 2 * ham).float()[keep], ref_span[:, :, t][keep])
        for tag in "abcd":
            init, recent, heavy, mode, depth = g[f"{name}_{tag}_params"]
            S = K.shape[2]
            ref_mask = torch.from_numpy(np.unpackbits(g[f"{name}_{tag}_mask"], axis=-1)[..., :S].astype(bool))
            mine = orc.compute_mask_multi(ref_span, int(init), int(recent), float(heavy), "simple" if mode == 0 else "thold", depth)
            # With fewer candidates than the heavy budget the reference's `indices[:heavy_budget]` runs into the
            # masked entries of the sort (hashattention_llama.py:437-438): window positions, already kept, and for
            # q_len > 1 positions after the query, which the additive causal mask (:598) keeps at zero weight.
            # Only the causal part of the mask has an effect, so only it is compared.
            q_len = Q.shape[2]
            causal = torch.tril(torch.ones(q_len, S), diagonal=S - q_len).bool()
            mine, ref_mask = mine & causal, ref_mask & causal
            score = torch.where(ref_span > -1e30, ref_span, torch.full_like(ref_span, -1e4))
            if mode == 0:
                # the reference's sort is unstable: equal up to the choice among equal scores ...
                assert orc.tie_invariant_equal(mine, ref_mask, score), (name, tag)
            else:
                assert torch.equal(mine, ref_mask), (name, tag)        # threshold mode keeps all ties: exact
            # ... and the index-set formulation used by the kernels agrees with the canonical mask row by row
            hb_abs = orc.heavy_count(S, float(heavy))
            for b in range(K.shape[0]):
                for t in range(q_len):
                    s_t = S - q_len + t + 1
                    ham_bt = ((32 - ref_span[b, :, t, :s_t]) / 2).round().long()
                    sel = orc.select_indices(ham_bt, s_t, int(init), int(recent), 0.0 if hb_abs == 0 else hb_abs + 0.5,
                                             "simple" if mode == 0 else "thold", int(depth))
                    assert torch.equal(orc.mask_from_indices(sel, S)[:, :s_t], mine[b, :, t, :s_t]), (name, tag, b, t)
                    assert not mine[b, :, t, s_t:].any()


def test_usa_state_dict_layout_matches_the_reference_checkpoints():
    """`load_usa` reads reference checkpoints by key: the hash module of this build must expose exactly the keys
    and shapes of the reference's `USA.state_dict()` (recorded in reference_vectors.npz), values interchangeable."""
    from hashattention._patched import USA
    g = np.load(os.path.join(HERE, "reference_vectors.npz"))
    keys = [str(k) for k in g["state_keys"]]
    usa = USA(4, 128, {"lth_int_dim": 32, "lth_final_dim": 32, "lth_thold": 0, "lth_num_layers": 3})
    sd = usa.state_dict()
    assert list(sd.keys()) == keys
    ref_sd = {k: torch.from_numpy(g[f"w{i}"]) for i, k in enumerate(keys)}
    for k in keys:
        assert sd[k].shape == ref_sd[k].shape, k
    usa.load_state_dict(ref_sd)                      # a reference state dict loads as is
    heads = usa.layers("k")
    assert torch.equal(heads[2][1][0], ref_sd["learning_to_hash_transformation_k.2.2.weight"])
    # and the ModuleList wrapping of load_usa gives the "{layer}." prefix of the shipped checkpoints
    ml = torch.nn.ModuleList([usa])
    assert list(ml.state_dict().keys())[0] == "0." + keys[0]


def test_training_side_of_the_oracle_matches_vectors_recorded_from_the_reference():
    """Soft-mode USA.forward, three train_step calls (weighted BCE, Adam) and the train branch's targets, as recorded
    from the reference's own code by tests/golden/make_reference_train_vectors.py."""
    g = np.load(os.path.join(HERE, "reference_train_vectors.npz"))
    K, Q = torch.from_numpy(g["K"]), torch.from_numpy(g["Q"])
    heads = _usa_heads(g)
    span, kt = orc.usa_forward_soft(K, Q, heads["k"], heads["q"], 0.0)
    assert (span - torch.from_numpy(g["soft_span"])).abs().max().item() < 1e-6
    assert (kt - torch.from_numpy(g["soft_k"])).abs().max().item() < 1e-6
    q_len, S = Q.shape[2], K.shape[2]
    assert (span[0, 0, 0, S - q_len + 1:] == 0).all()                  # non-causal entries: sigmoid(finfo.min) = 0 exactly
    # three optimizer steps from the recorded start
    leaf = _usa_heads(g, leaf=True)
    params = [t for side in ("k", "q") for head in leaf[side] for wb in head for t in wb]
    alpha, beta = g["bce_alpha_beta"]
    loss_fn = orc.weighted_bce(float(alpha), float(beta))
    opt = torch.optim.Adam(params, lr=0.001)
    target = torch.from_numpy(g["target"].astype(np.float32))
    mask = torch.from_numpy(g["target_mask"])
    losses = [orc.train_step(K, Q, target, mask, leaf["k"], leaf["q"], loss_fn, opt) for _ in range(3)]
    assert np.abs(np.array(losses) - g["losses"]).max() < 1e-5 and losses[2] < losses[0]
    after = _usa_heads(g, prefix="w_after")
    for side in ("k", "q"):
        for mine, ref in zip(leaf[side], after[side]):
            for (w, b), (wr, br) in zip(mine, ref):
                assert (w.detach() - wr).abs().max().item() < 2e-6 and (b.detach() - br).abs().max().item() < 2e-6
    assert (leaf["k"][0][0][0].detach() - heads["k"][0][0][0]).abs().max().item() > 1e-4       # the weights did move
    # the loss alone, from its definition: mean of -w [y log p + (1 - y) log(1 - p)], positives weighted S * beta + alpha
    p0 = span.masked_fill(~mask, 0).double()
    y = target.double()
    wgt = torch.where(y > 0, torch.tensor(S * float(beta) + float(alpha), dtype=torch.float64), torch.tensor(1.0, dtype=torch.float64))
    by_hand = -(wgt * (y * torch.log(p0).clamp(min=-100) + (1 - y) * torch.log(1 - p0).clamp(min=-100))).mean().item()
    assert abs(by_hand - g["losses"][0]) < 1e-5
    # targets of the train branch
    d = 128
    hs = torch.from_numpy(g["lc_hidden"])
    qw = torch.from_numpy(g["lc_q_weight"])
    keys = torch.from_numpy(g["lc_keys"].astype(np.float32))
    cos, sin = torch.from_numpy(g["lc_cos"]), torch.from_numpy(g["lc_sin"])
    q = (hs @ qw.t()).view(1, hs.shape[1], -1, d).transpose(1, 2)
    q, _ = orc.apply_rotary_pos_emb(q, q, cos, sin)
    assert (q - torch.from_numpy(g["lc_Q"])).abs().max().item() < 1e-5
    init, recent = (int(x) for x in g["lc_params"])
    tgt, cand = orc.recall_targets(q, keys, init, recent)
    S2 = keys.shape[2]
    assert np.array_equal(np.packbits(cand.numpy(), axis=-1), g["lc_mask"])
    assert np.array_equal(np.packbits(tgt.numpy().astype(bool), axis=-1), g["lc_target"])
    assert int(tgt.sum()) == 32 * q.shape[1] * q.shape[2] and not tgt[..., ~cand[-1]].bool()[..., -1, :].any() and S2 == 1024


def _center_heads(g):
    keys = [str(k) for k in g["center_keys"]]
    sd = {k: torch.from_numpy(g[f"center_w{i}"]) for i, k in enumerate(keys)}
    return {side: [[(sd[f"learning_to_hash_transformation_{side}.{h}.{l}.weight"], sd[f"learning_to_hash_transformation_{side}.{h}.{l}.bias"])
                    for l in (0, 2, 4)] for h in range(3)] for side in ("k", "q")}


def _lsh_heads(g):
    return [[(torch.from_numpy(g[f"lsh_w{2 * h}"]), torch.from_numpy(g[f"lsh_w{2 * h + 1}"]))] for h in range(3)]


def _span_mismatches(mine, want):
    """Entries of two hard spans that differ: a logit within round-off of zero may change one sign, i.e. 2 in the span."""
    diff = (mine - want).abs()
    assert diff.max().item() <= 2.0
    return int((diff > 0).sum())


def test_center_and_lsh_variants_of_the_oracle_match_vectors_recorded_from_the_reference():
    """The CENTER switch and the LSH baseline, hard and soft mode, as recorded from the reference's own code by
    tests/golden/make_reference_lsh_center_vectors.py (two batch entries: pins that the statistics run over batch and
    positions of one head)."""
    g = np.load(os.path.join(HERE, "reference_lsh_center_vectors.npz"))
    K, Q = torch.from_numpy(g["K"]), torch.from_numpy(g["Q"])
    ch = _center_heads(g)
    span, ks = orc.usa_forward_hard(K, Q, ch["k"], ch["q"], center=True)
    want = torch.from_numpy(g["center_hard_span"])
    assert _span_mismatches(span, want) == 0
    assert torch.equal(ks.to(torch.int8), torch.from_numpy(g["center_hard_k"]))
    # the switch matters on these inputs, and leaving it out reproduces the recorded plain spans
    plain, _ = orc.usa_forward_hard(K, Q, ch["k"], ch["q"])
    assert _span_mismatches(plain, torch.from_numpy(g["plain_hard_span"])) == 0
    assert (plain != span).float().mean().item() > 0.5
    soft, kt = orc.usa_forward_soft(K, Q, ch["k"], ch["q"], 0.0, center=True)
    assert (soft - torch.from_numpy(g["center_soft_span"])).abs().max().item() < 1e-5
    assert (kt - torch.from_numpy(g["center_soft_k"])).abs().max().item() < 1e-5
    # a plausible mistake - statistics per batch entry instead of over the batch - does not reproduce the vectors
    wrong = torch.cat([orc.usa_forward_hard(K[i:i + 1], Q[i:i + 1], ch["k"], ch["q"], center=True)[0] for i in range(2)])
    assert (wrong != want).any()

    # ---- LSH baseline: state-dict layout (three prefixes over the same tensors), lift, shared projection
    keys = [str(k) for k in g["lsh_keys"]]
    assert keys[:2] == ["learning_to_hash_transformation.0.1.weight", "learning_to_hash_transformation.0.1.bias"]
    assert len(keys) == 18 and keys[6].startswith("learning_to_hash_transformation_k.") and keys[12].startswith("learning_to_hash_transformation_q.")
    lh = _lsh_heads(g)
    assert lh[0][0][0].shape == (32, 129)
    span, ks = orc.usa_forward_hard(K, Q, lh, lh, lsh=True)
    want = torch.from_numpy(g["lsh_hard_span"])
    assert _span_mismatches(span, want) == 0
    assert torch.equal(ks.to(torch.int8), torch.from_numpy(g["lsh_hard_k"]))
    assert torch.equal(torch.from_numpy(g["lsh_k_embedding_hard"]), torch.from_numpy(g["lsh_hard_k"]))
    soft, kt = orc.usa_forward_soft(K, Q, lh, lh, 0.0, lsh=True)
    assert (soft - torch.from_numpy(g["lsh_soft_span"])).abs().max().item() < 1e-5
    assert (kt - torch.from_numpy(g["lsh_soft_k"])).abs().max().item() < 1e-4
    # the lift by its definition: every lifted vector of a head has the same norm, the head's largest norm + 1e-3
    lifted = orc.lift_heads(K)
    top = K.norm(dim=-1).amax(dim=(0, 2)) + 1e-3
    assert (lifted.norm(dim=-1) - top[None, :, None]).abs().max().item() < 1e-4
    assert torch.equal(lifted[..., :128], K)
    # a plausible mistake - one largest norm for all heads - does not reproduce the vectors
    flat = orc.lift_one_head(K)
    wrong_logits = orc.usa_logits(flat, lh)
    right_logits = orc.usa_logits(lifted, lh)
    assert (torch.sign(wrong_logits) != torch.sign(right_logits)).any()


def test_module_variants_expose_the_reference_layout_and_soft_scores():
    """The shipped `USA` in its LSH and CENTER variants: state-dict keys of the reference, a recorded state dict loads, and
    the soft mode (torch code, runs without a GPU) reproduces the recorded scores."""
    from hashattention._patched import USA, lift_to_sphere
    g = np.load(os.path.join(HERE, "reference_lsh_center_vectors.npz"))
    K, Q = torch.from_numpy(g["K"]), torch.from_numpy(g["Q"])
    lsh = USA(3, 128, {"lth_int_dim": 128, "lth_final_dim": 32, "lth_thold": 0, "lth_num_layers": 0})
    lsh.center = False
    keys = [str(k) for k in g["lsh_keys"]]
    assert list(lsh.state_dict().keys()) == keys
    lsh.load_state_dict({k: torch.from_numpy(g[f"lsh_w{i % 6}"]) for i, k in enumerate(keys)})
    assert lsh.rehash_every_step and lsh.kernel_num_layers == 1
    assert lsh.kernel_layers("k")[0][0][0].shape == (32, 132) and (lsh.kernel_layers("q")[2][0][0][:, 129:] == 0).all()
    with torch.no_grad():
        soft, kt = lsh(K, Q)
    assert (soft - torch.from_numpy(g["lsh_soft_span"])).abs().max().item() < 1e-5
    assert (kt - torch.from_numpy(g["lsh_soft_k"])).abs().max().item() < 1e-4
    # the batched lift equals the oracle's head-by-head one, padding aside
    mine = lift_to_sphere(K, 3)
    assert torch.equal(mine[..., :129], orc.lift_heads(K)) and (mine[..., 129:] == 0).all()

    usa = USA(3, 128, {"lth_int_dim": 32, "lth_final_dim": 32, "lth_thold": 0, "lth_num_layers": 3})
    ckeys = [str(k) for k in g["center_keys"]]
    usa.load_state_dict({k: torch.from_numpy(g[f"center_w{i}"]) for i, k in enumerate(ckeys)})
    usa.center = True
    assert usa.rehash_every_step
    with torch.no_grad():
        soft, kt = usa(K, Q)
        Kh, Qh = usa.hash_inputs(K, Q)
    assert (soft - torch.from_numpy(g["center_soft_span"])).abs().max().item() < 1e-5
    Ko, Qo = orc.standardise_by_keys(K, Q)
    assert (Kh - Ko).abs().max().item() < 1e-5 and (Qh - Qo).abs().max().item() < 1e-5
    # keys of KV heads against queries of more heads: statistics of KV head i // group
    Kg, Qg = K[:, :1], Q
    Kh, Qh = usa.hash_inputs(Kg, Qg)
    Ko, Qo = orc.standardise_by_keys(Kg.expand(-1, 3, -1, -1), Qg)
    assert (Qh - Qo).abs().max().item() < 1e-5 and (Kh - Ko[:, :1]).abs().max().item() < 1e-5
