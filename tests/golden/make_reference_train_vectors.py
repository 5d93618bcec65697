"""One-off generator of golden vectors for the training side, from the reference's own code (build container only).

Imports /root/reference/hashattention/hashattention_llama.py on the CPU and records, for small seeded inputs,
  * `USA.forward(K, Q)` in soft mode (tanh embeddings, sigmoid(span - thold), non-causal entries at sigmoid(finfo.min) = 0),
  * three consecutive `LlamaAttention_heavy_hitter.train_step` calls (weighted-BCE loss of the training script, Adam):
    the loss before every step and the state dict after the last one,
  * the train branch of `usa_local_compute`: which (target, target_mask) it hands to `train_step` for a given layer input
    (true-logit top-32 among the candidates [init, pos - recent]).
Nothing in the reference's tests pins these; the outputs are committed as data: tests/golden/reference_train_vectors.npz.

    python tests/golden/make_reference_train_vectors.py
"""
import os
import sys
import types

import numpy as np
import torch

REF = "/root/reference"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_train_vectors.npz")


def bce_loss(alpha, beta):
    # the loss of the training script (train_hashattention.py:88-95), restated
    def f(yhat, y):
        w = y.shape[-1] * beta + alpha
        weight = y * (w - 1) + torch.ones_like(y)
        return torch.nn.functional.binary_cross_entropy(yhat.reshape(-1), y.reshape(-1), weight=weight.reshape(-1))
    return f


def main():
    sys.dont_write_bytecode = True      # the reference tree is read-only: no __pycache__ beside its sources
    sys.path.insert(0, REF)
    from hashattention import hashattention_llama as ref   # prints "CENTER 0"

    out = {}
    torch.manual_seed(4321)
    H, d, S, q_len = 2, 128, 48, 6
    cfg = {"lth_int_dim": 32, "lth_final_dim": 32, "lth_thold": 0, "lth_num_layers": 3}
    usa = ref.USA(H, d, cfg)
    sd = usa.state_dict()
    out["state_keys"] = np.array(list(sd.keys()))
    for i, v in enumerate(sd.values()):
        out[f"w{i}"] = v.detach().clone().numpy()
    K = torch.randn(1, H, S, d)
    Q = torch.randn(1, H, q_len, d)
    out["K"], out["Q"] = K.numpy(), Q.numpy()
    span, ktanh = usa(K, Q)                         # soft mode is the default
    out["soft_span"] = span.detach().numpy()
    out["soft_k"] = ktanh.detach().numpy()

    # targets: 5 random candidates per row inside the causal region, mask = causal region minus a recent window of 3
    causal = torch.tril(torch.ones(q_len, S), diagonal=S - q_len - 3).bool()
    target = torch.zeros(1, H, q_len, S)
    g = torch.Generator().manual_seed(7)
    for h in range(H):
        for i in range(q_len):
            n = int(causal[i].sum())
            pick = torch.randperm(n, generator=g)[:5]
            target[0, h, i, pick] = 1.0
    out["target"] = target.numpy().astype(np.uint8)
    out["target_mask"] = causal.numpy()
    alpha, beta = 1.0, 0.5
    out["bce_alpha_beta"] = np.array([alpha, beta])
    loss_fn = bce_loss(alpha, beta)
    opt = torch.optim.Adam(usa.parameters(), lr=0.001)
    ns = types.SimpleNamespace(usa_module=usa, tr_loss_func=loss_fn, tr_optimizer=opt, layer_idx=0)
    losses = []
    for _ in range(3):
        with torch.no_grad():
            s, _ = usa(K, Q)
            losses.append(loss_fn(s.masked_fill(torch.logical_not(causal), 0), target).item())
        ref.LlamaAttention_heavy_hitter.train_step(ns, K, Q, target, causal)
    out["losses"] = np.array(losses)
    for i, v in enumerate(usa.state_dict().values()):
        out[f"w_after{i}"] = v.detach().numpy()

    # ---- train branch of usa_local_compute: the (target, mask) handed to train_step
    torch.manual_seed(99)
    H2, Hkv2, S2, q2, hidden = 2, 1, 1024, 4, 64
    q_proj = torch.nn.Linear(hidden, H2 * d, bias=False)
    k_proj = torch.nn.Linear(hidden, Hkv2 * d, bias=False)
    hs = torch.randn(1, q2, hidden)
    keys = torch.randn(1, Hkv2, S2, d).half().float()     # fp16-exact values: stored as fp16 without loss
    ang = torch.randn(1, q2, d // 2)
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1), torch.cat([ang.sin(), ang.sin()], -1)
    got = {}

    def capture(Kx, Qx, tgt, msk):
        got["K"], got["Q"], got["target"], got["mask"] = Kx, Qx, tgt, msk

    layer = types.SimpleNamespace(layer_idx=0, q_proj=q_proj, k_proj=k_proj, num_heads=H2, head_dim=d, num_key_value_heads=Hkv2,
                                  num_key_value_groups=H2 // Hkv2, init_budget=16, recent_budget=32, train_usa=True,
                                  train_step=capture)
    cache = types.SimpleNamespace(key_cache=[keys])
    with torch.no_grad():
        ref.LlamaAttention_heavy_hitter.usa_local_compute(layer, hs, None, None, cache, (cos, sin))
    out["lc_hidden"], out["lc_keys"] = hs.numpy(), keys.numpy().astype(np.float16)
    out["lc_q_weight"], out["lc_k_weight"] = q_proj.weight.detach().numpy(), k_proj.weight.detach().numpy()
    out["lc_cos"], out["lc_sin"] = cos.numpy(), sin.numpy()
    out["lc_params"] = np.array([16, 32])
    out["lc_target"] = np.packbits(got["target"].numpy().astype(bool), axis=-1)
    out["lc_mask"] = np.packbits(got["mask"].numpy(), axis=-1)
    out["lc_Q"] = got["Q"].numpy()
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
