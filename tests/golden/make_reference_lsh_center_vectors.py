"""One-off generator of golden vectors for the two hash variants whose codes depend on the whole cache, from the
reference's own code (build container only).

Imports /root/reference/hashattention/hashattention_llama.py on the CPU and records, for small seeded fp32 inputs with two
batch entries (so that statistics over batch AND positions are pinned):
  * the 3-layer `USA` with its `center` attribute set (the CENTER switch): `forward(K, Q, hard=True)` and soft mode;
  * the LSH baseline (`lth_num_layers = 0`): its state-dict keys (every tensor appears under three prefixes; one copy is kept), `forward` in hard
    and soft mode, and `k_embedding(K, hard=True)`.
Nothing in the reference's tests pins these; the outputs are committed as data: tests/golden/reference_lsh_center_vectors.npz.

    python tests/golden/make_reference_lsh_center_vectors.py
"""
import os
import sys

import numpy as np
import torch

REF = "/root/reference"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_lsh_center_vectors.npz")


def main():
    sys.dont_write_bytecode = True      # the reference tree is read-only: no __pycache__ beside its sources
    sys.path.insert(0, REF)
    from hashattention import hashattention_llama as ref   # prints "CENTER 0"

    out = {}
    torch.manual_seed(2024)
    b, H, d, S, q_len = 2, 3, 128, 40, 3
    # keys with a per-feature offset and spread, so that standardising changes signs
    K = torch.randn(b, H, S, d) * (0.5 + torch.rand(1, H, 1, d)) + torch.randn(1, H, 1, d)
    Q = torch.randn(b, H, q_len, d)
    out["K"], out["Q"] = K.numpy(), Q.numpy()

    usa = ref.USA(H, d, {"lth_int_dim": 32, "lth_final_dim": 32, "lth_thold": 0, "lth_num_layers": 3})
    usa.center = True
    out["center_keys"] = np.array(list(usa.state_dict().keys()))
    for i, v in enumerate(usa.state_dict().values()):
        out[f"center_w{i}"] = v.detach().clone().numpy()
    with torch.no_grad():
        span, ksign = usa(K, Q, hard=True)
        out["center_hard_span"], out["center_hard_k"] = span.numpy(), ksign.numpy().astype(np.int8)
        soft, ktanh = usa(K, Q)
        out["center_soft_span"], out["center_soft_k"] = soft.numpy(), ktanh.numpy()
        usa.center = False
        plain, _ = usa(K, Q, hard=True)
        out["plain_hard_span"] = plain.numpy()          # the same weights without the switch: shows the switch matters

    lsh = ref.USA(H, d, {"lth_int_dim": 128, "lth_final_dim": 32, "lth_thold": 0, "lth_num_layers": 0})
    lsh.center = False
    sd = lsh.state_dict()
    out["lsh_keys"] = np.array(list(sd.keys()))
    base = "learning_to_hash_transformation."
    for side in ("k", "q"):                                 # the three prefixes name the same tensors: keep one copy
        for key, v in sd.items():
            if key.startswith(base):
                assert torch.equal(v, sd[key.replace(base, f"learning_to_hash_transformation_{side}.")])
    for i, (key, v) in enumerate((k, v) for k, v in sd.items() if k.startswith(base)):
        out[f"lsh_w{i}"] = v.detach().clone().numpy()
    with torch.no_grad():
        span, ksign = lsh(K, Q, hard=True)
        out["lsh_hard_span"], out["lsh_hard_k"] = span.numpy(), ksign.numpy().astype(np.int8)
        soft, ktanh = lsh(K, Q)
        out["lsh_soft_span"], out["lsh_soft_k"] = soft.numpy(), ktanh.numpy()
        out["lsh_k_embedding_hard"] = lsh.k_embedding(K, hard=True).numpy().astype(np.int8)
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
