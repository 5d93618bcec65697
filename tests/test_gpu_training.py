"""The training side of the drop-in on a GPU: soft-mode `USA.forward`, `train_step`, the train branch of
`usa_local_compute` and the KV offload policy, against the vectors recorded from the reference's own code
(tests/golden/make_reference_train_vectors.py) and against the oracle's restatement (hashattention_llama.py:151-200,
:304-316, :356-371, :495-511)."""
import os

import numpy as np
import pytest
import torch
from transformers import DynamicCache, LlamaConfig, LlamaForCausalLM

from hashattention import hashattention_llama as hl
from hashattention._patched import USA, HeavyHitterMixin
from oracle import hashattn_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_train_vectors.npz")
USA_CFG = dict(lth_init_dim=128, lth_final_dim=32, lth_thold=0, lth_num_layers=3, init_budget=8, heavy_budget=0.125,
               recent_budget=8, usa_retrieve_depth=6, usa_eval_mode="simple")


def _recorded_usa(g, prefix="w"):
    keys = [str(k) for k in g["state_keys"]]
    usa = USA(2, 128, {"lth_int_dim": 32, "lth_final_dim": 32, "lth_thold": 0, "lth_num_layers": 3})
    usa.load_state_dict({k: torch.from_numpy(g[f"{prefix}{i}"]) for i, k in enumerate(keys)})
    return usa.to(DEV)


class _Layer(HeavyHitterMixin):
    """The mixin's training state without a model around it."""
    def __init__(self, usa, loss, opt, layer_idx=0):
        self.usa_module, self.tr_loss_func, self.tr_optimizer, self.layer_idx = usa, loss, opt, layer_idx
        self._hash_layer = None
        self.last_train_loss = None


def test_soft_forward_and_train_steps_match_the_reference_vectors():
    print("\n[case] soft forward + 3 train steps vs recorded reference", flush=True)
    g = np.load(GOLDEN)
    usa = _recorded_usa(g)
    K, Q = torch.from_numpy(g["K"]).to(DEV), torch.from_numpy(g["Q"]).to(DEV)
    with torch.no_grad():
        span, kt = usa(K, Q)                                       # soft mode is the default, as in the reference
    assert (span.cpu() - torch.from_numpy(g["soft_span"])).abs().max().item() < 1e-5
    assert (kt.cpu() - torch.from_numpy(g["soft_k"])).abs().max().item() < 1e-5
    assert (usa.k_embedding(K).cpu() - torch.from_numpy(g["soft_k"])).abs().max().item() < 1e-5
    q_len, S = Q.shape[2], K.shape[2]
    assert (span[0, 0, 0, S - q_len + 1:] == 0).all()
    alpha, beta = (float(x) for x in g["bce_alpha_beta"])
    layer = _Layer(usa, orc.weighted_bce(alpha, beta), torch.optim.Adam(usa.parameters(), lr=0.001))
    target = torch.from_numpy(g["target"].astype(np.float32)).to(DEV)
    mask = torch.from_numpy(g["target_mask"]).to(DEV)
    losses = []
    with torch.inference_mode():                                   # the generation loop the reference trains under
        for _ in range(3):
            layer.train_step(K, Q, target, mask)
            losses.append(layer.last_train_loss.item())
    print("losses", losses, "recorded", g["losses"].tolist(), flush=True)
    assert np.abs(np.array(losses) - g["losses"]).max() < 1e-4
    want = _recorded_usa(g, prefix="w_after").state_dict()
    diffs = torch.cat([(v - want[k]).abs().flatten() for k, v in usa.state_dict().items()])
    start = _recorded_usa(g).state_dict()
    moved = torch.cat([(v - start[k]).abs().flatten() for k, v in usa.state_dict().items()])
    print(f"after 3 Adam steps: max difference {diffs.max().item():.2e}, mean movement {moved.mean().item():.2e}", flush=True)
    # Adam divides by the gradient's magnitude, so a parameter whose gradient is at rounding level can land elsewhere
    assert (diffs < 1e-4).float().mean().item() > 0.999 and diffs.median().item() < 1e-6
    assert moved.mean().item() > 1e-3


def test_soft_forward_matches_the_oracle_on_other_shapes():
    print("\n[case] soft forward vs oracle, 2-layer / 64-bit / thold", flush=True)
    torch.manual_seed(3)
    for nl, D, thold in ((2, 64, 0.5), (1, 32, 0.0), (3, 32, 1.0)):
        usa = USA(3, 128, {"lth_int_dim": 128, "lth_final_dim": D, "lth_thold": thold, "lth_num_layers": nl}).to(DEV)
        K, Q = torch.randn(2, 3, 40, 128), torch.randn(2, 3, 5, 128)
        heads = {s: [[(w.detach().cpu(), b.detach().cpu()) for w, b in h] for h in usa.layers(s)] for s in "kq"}
        want, wk = orc.usa_forward_soft(K, Q, heads["k"], heads["q"], thold)
        with torch.no_grad():
            got, gk = usa(K.to(DEV), Q.to(DEV))
        assert (got.cpu() - want).abs().max().item() < 1e-5 and (gk.cpu() - wk).abs().max().item() < 1e-5
    # gradients reach the per-head modules: against autograd through the oracle's per-head loop
    leaf = {s: [[(w.detach().cpu().requires_grad_(), b.detach().cpu().requires_grad_()) for w, b in h] for h in usa.layers(s)] for s in "kq"}
    orc.usa_forward_soft(K, Q, leaf["k"], leaf["q"], thold)[0].square().sum().backward()
    usa(K.to(DEV), Q.to(DEV))[0].square().sum().backward()
    for s in "kq":
        for h, head in enumerate(usa.layers(s)):
            for l, (w, b) in enumerate(head):
                assert (w.grad.cpu() - leaf[s][h][l][0].grad).abs().max().item() < 1e-4
                assert (b.grad.cpu() - leaf[s][h][l][1].grad).abs().max().item() < 1e-4


def _tiny_llama():
    cfg = LlamaConfig(hidden_size=64, intermediate_size=128, num_hidden_layers=1, num_attention_heads=2, num_key_value_heads=1,
                      head_dim=128, vocab_size=64, max_position_embeddings=4096)
    for k, v in USA_CFG.items():
        setattr(cfg, k, v)
    return cfg


def test_train_branch_hands_the_reference_targets_to_train_step():
    print("\n[case] usa_local_compute train branch vs recorded reference", flush=True)
    g = np.load(GOLDEN)
    cfg = _tiny_llama()
    cfg.init_budget, cfg.recent_budget = (int(x) for x in g["lc_params"])
    layer = hl.LlamaAttention_heavy_hitter(cfg, 0).to(DEV)
    with torch.no_grad():
        layer.q_proj.weight.copy_(torch.from_numpy(g["lc_q_weight"]))
        layer.k_proj.weight.copy_(torch.from_numpy(g["lc_k_weight"]))
    layer.usa_module = USA(2, 128, {"lth_int_dim": 32, "lth_final_dim": 32, "lth_thold": 0, "lth_num_layers": 3}).to(DEV)
    layer.train_usa = True
    keys = torch.from_numpy(g["lc_keys"].astype(np.float32)).to(DEV)
    cache = DynamicCache()
    cache.update(keys, torch.zeros_like(keys), 0)
    got = {}
    layer.train_step = lambda K, Q, target, mask: got.update(K=K, Q=Q, target=target, mask=mask)
    hs = torch.from_numpy(g["lc_hidden"]).to(DEV)
    cos, sin = torch.from_numpy(g["lc_cos"]).to(DEV), torch.from_numpy(g["lc_sin"]).to(DEV)
    with torch.no_grad():
        layer.usa_local_compute(hs, None, None, cache, (cos, sin))
    assert (got["Q"].cpu() - torch.from_numpy(g["lc_Q"])).abs().max().item() < 1e-4
    assert got["K"].shape == (1, 2, 1024, 128) and torch.equal(got["K"][0, 0], got["K"][0, 1])      # KV head repeated per query head
    assert np.array_equal(np.packbits(got["mask"].cpu().numpy(), axis=-1), g["lc_mask"])
    assert np.array_equal(np.packbits(got["target"].cpu().numpy().astype(bool), axis=-1), g["lc_target"])
    # a cache length that is not a multiple of 1024 is skipped (reference :329-332)
    got.clear()
    cache2 = DynamicCache()
    cache2.update(keys[:, :, :1000], torch.zeros_like(keys[:, :, :1000]), 0)
    layer.usa_local_compute(hs, None, None, cache2, (cos, sin))
    assert not got


def test_training_through_the_model_api_then_decoding_with_the_trained_hash():
    print("\n[case] convert_usa(train_usa=True) + set_train_usa_mode, then eval decode", flush=True)
    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                      head_dim=128, vocab_size=256, max_position_embeddings=4096)
    for k, v in USA_CFG.items():
        setattr(cfg, k, v)
    model = LlamaForCausalLM(cfg).bfloat16().to(DEV)            # the training script's setting: model and hash in bf16
    usa = hl.load_usa(cfg, None).bfloat16()
    model = hl.convert_usa(model, cfg, usa, collect_stats=True, train_usa=True)
    before = [p.detach().clone() for p in usa.parameters()]
    opt = torch.optim.Adam(usa.parameters(), lr=0.001)
    hl.set_train_usa_mode(model, orc.weighted_bce(1.0, 0.5), opt)
    ids = torch.randint(0, cfg.vocab_size, (1, 1024 + 5), generator=torch.Generator().manual_seed(1)).to(DEV)
    layers = [m for m in model.modules() if isinstance(m, hl.LlamaAttention_heavy_hitter)]
    losses = []
    for _ in range(4):                                   # the same prompt four times: the loss of every layer must fall
        cache = DynamicCache()
        with torch.inference_mode():
            model(ids[:, :1024], past_key_values=cache, use_cache=True)       # cache length 1024: one train step per layer
        losses.append([m.last_train_loss.item() for m in layers])
        hl.reset_usa(model)
    print("train losses per pass", losses, flush=True)
    assert all(np.isfinite(l).all() for l in losses) and all(losses[-1][i] < losses[0][i] for i in range(len(layers)))
    assert any((p.detach() - b).abs().max().item() > 0 for p, b in zip(usa.parameters(), before))
    # back to inference: decode steps run on the kernels with the trained weights
    hl.set_eval_usa_mode(model)
    cache = DynamicCache()
    with torch.no_grad():
        model(ids[:, :1024], past_key_values=cache, use_cache=True)
        for t in range(3):
            out = model(ids[:, 1024 + t:1025 + t], past_key_values=cache, use_cache=True).logits
            assert torch.isfinite(out).all()
    m0 = layers[0]
    assert m0._hash_layer is not None and m0._hash_layer.n_cached == 1027
    # the bit-cache was built from the updated parameters
    keys = cache.layers[0].keys
    codes = torch.zeros_like(m0._hash_layer.codes[:, :, :1027])
    from hashattention import _ops
    w = _ops.pack_usa_weights(m0.usa_module.layers("k"), keys.device)
    _ops.encode_pack(keys, w, 3, 128, 32, codes, 0, None, m0.usa_module.arith)
    agree = (codes == m0._hash_layer.codes[:, :, :1027]).float().mean().item()
    assert agree > 0.99, agree                          # the MFMA bulk encoder may flip bits of near-zero logits


def test_kv_offload_policy_moves_the_cache_and_changes_nothing():
    print("\n[case] KV offload policy", flush=True)
    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                      head_dim=128, vocab_size=256, max_position_embeddings=4096)
    for k, v in USA_CFG.items():
        setattr(cfg, k, v)
    model = LlamaForCausalLM(cfg).to(DEV)
    usa = hl.load_usa(cfg, None)
    model = hl.convert_usa(model, cfg, usa, collect_stats=False, train_usa=False).float()
    layers = [m for m in model.modules() if isinstance(m, hl.LlamaAttention_heavy_hitter)]
    assert all(m.offloading_length is None for m in layers)          # off unless asked for
    ids = torch.randint(0, cfg.vocab_size, (1, 203), generator=torch.Generator().manual_seed(2)).to(DEV)

    def run(offload):
        for m in layers:
            m.offloading_length = offload
        hl.reset_usa(model)
        cache = DynamicCache()
        outs = []
        with torch.no_grad():
            model(ids[:, :200], past_key_values=cache, use_cache=True)
            for t in range(3):
                outs.append(model(ids[:, 200 + t:201 + t], past_key_values=cache, use_cache=True).logits.float().cpu())
        return outs, cache

    plain, cache_a = run(None)
    assert cache_a.layers[0].keys.is_cuda
    off, cache_b = run(201)                                            # from 201 cached tokens on, the cache lives on the host
    assert not cache_b.layers[0].keys.is_cuda and not cache_b.layers[1].values.is_cuda
    for a, b in zip(plain, off):
        assert torch.equal(a, b)
