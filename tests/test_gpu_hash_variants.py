"""The two hash variants whose codes depend on the whole cache - the CENTER switch (keys and queries standardised with the
statistics of the cached keys, hashattention_llama.py:163-167) and the LSH baseline (`lth_num_layers = 0`, :75-84,
:130-139) - on the GPU: the module API against vectors recorded from the reference's own code, and a patched model
against the same model on the CPU running the oracle's restatement of the reference's decode branch."""
import copy
import os

import numpy as np
import pytest
import torch
from transformers import LlamaConfig, LlamaForCausalLM

from hashattention import hashattention_llama as hl
from hashattention._patched import USA
from tests.test_gpu_model_api import _config, _oracle_forward, _run

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_lsh_center_vectors.npz")


def _span_mismatches(mine, want):
    diff = (mine.float().cpu() - want).abs()
    assert diff.max().item() <= 2.0          # one sign of one code may differ where a logit is within round-off of zero
    return int((diff > 0).sum())


def test_module_api_reproduces_vectors_recorded_from_the_reference():
    print("\n[case] USA.forward(hard) with CENTER / LSH against recorded vectors", flush=True)
    g = np.load(GOLDEN)
    K, Q = torch.from_numpy(g["K"]).to(DEV), torch.from_numpy(g["Q"]).to(DEV)

    usa = USA(3, 128, {"lth_int_dim": 32, "lth_final_dim": 32, "lth_thold": 0, "lth_num_layers": 3})
    keys = [str(k) for k in g["center_keys"]]
    usa.load_state_dict({k: torch.from_numpy(g[f"center_w{i}"]) for i, k in enumerate(keys)})
    usa = usa.to(DEV)
    usa.center = True
    with torch.no_grad():
        span, ksign = usa(K, Q, hard=True)
    n = _span_mismatches(span, torch.from_numpy(g["center_hard_span"]))
    flips = int((ksign.cpu().to(torch.int8) != torch.from_numpy(g["center_hard_k"])).sum())
    print(f"  center: span entries differing {n}, key signs differing {flips}", flush=True)
    assert n <= 6 and flips <= 2
    usa.center = False
    with torch.no_grad():
        plain, _ = usa(K, Q, hard=True)
    assert _span_mismatches(plain, torch.from_numpy(g["plain_hard_span"])) <= 6

    lsh = USA(3, 128, {"lth_int_dim": 128, "lth_final_dim": 32, "lth_thold": 0, "lth_num_layers": 0})
    lkeys = [str(k) for k in g["lsh_keys"]]
    lsh.load_state_dict({k: torch.from_numpy(g[f"lsh_w{i % 6}"]) for i, k in enumerate(lkeys)})
    lsh = lsh.to(DEV)
    lsh.center = False
    with torch.no_grad():
        span, ksign = lsh(K, Q, hard=True)
        kemb = lsh.k_embedding(K, hard=True)
        soft, _ = lsh(K, Q)
    n = _span_mismatches(span, torch.from_numpy(g["lsh_hard_span"]))
    flips = int((ksign.cpu().to(torch.int8) != torch.from_numpy(g["lsh_hard_k"])).sum())
    print(f"  lsh: span entries differing {n}, key signs differing {flips}", flush=True)
    assert n <= 6 and flips <= 2
    assert int((kemb.cpu().to(torch.int8) != torch.from_numpy(g["lsh_k_embedding_hard"])).sum()) <= 2
    assert (soft.cpu() - torch.from_numpy(g["lsh_soft_span"])).abs().max().item() < 1e-4


@pytest.mark.parametrize("variant", ["center", "lsh"])
def test_patched_model_with_a_cache_dependent_hash(variant):
    print(f"\n[case] patched model, hash variant {variant}", flush=True)
    torch.manual_seed(5)
    cfg = _config(LlamaConfig)
    if variant == "lsh":
        cfg.lth_num_layers = 0
    model = LlamaForCausalLM(cfg).bfloat16().float()
    ref = copy.deepcopy(model)
    usa = hl.load_usa(cfg, None)
    for m in usa:
        m.center = variant == "center"
        assert m.rehash_every_step
    model = hl.convert_usa(model.to(DEV), cfg, usa, collect_stats=False, train_usa=False).float()
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
    for li, layer in enumerate(ref.model.layers):
        _oracle_forward(layer.self_attn, usa[li], cfg, apply_rotary_pos_emb, **{variant: True})
    ids = torch.randint(0, cfg.vocab_size, (2, 200 + 1 + 1 + 5 + 1), generator=torch.Generator().manual_seed(2))
    steps = [1, 1, 5, 1]
    got = _run(model, ids.to(DEV), steps)
    want = _run(ref, ids, steps)
    for a, b in zip(got, want):
        err = (a - b).abs().max().item()
        print(f"  max |logit difference| {err:.2e}", flush=True)
        assert a.shape == b.shape and err < 2e-3, err
    # the codes were rebuilt at every step: the bit-cache holds exactly the keys of the last call
    assert model.model.layers[0].self_attn._hash_layer.n_cached == ids.shape[1]
    # compute_mask_multi of the patched layer agrees with the oracle's mask in this variant too
    layer = model.model.layers[0].self_attn
    from oracle import hashattn_oracle as orc
    K = torch.randn(1, 2, 300, 128, generator=torch.Generator().manual_seed(9))
    Q = torch.randn(1, 4, 3, 128, generator=torch.Generator().manual_seed(10))
    mask = layer.compute_mask_multi(K.to(DEV).repeat_interleave(2, dim=1), Q.to(DEV)).cpu()
    heads = lambda mods: [[(m.weight.detach().float().cpu(), m.bias.detach().float().cpu()) for m in seq if isinstance(m, torch.nn.Linear)]
                          for seq in mods]
    u = usa[0]
    span, _ = orc.usa_forward_hard(K.repeat_interleave(2, dim=1), Q, heads(u.learning_to_hash_transformation_k),
                                   heads(u.learning_to_hash_transformation_q), **{variant: True})
    want_mask = orc.compute_mask_multi(span, cfg.init_budget, cfg.recent_budget, cfg.heavy_budget)
    causal = torch.tril(torch.ones(3, 300), diagonal=300 - 3).bool()
    assert torch.equal(mask & causal, want_mask & causal)
