"""`load_usa(config, path)` with real files (reference: hashattention/hashattention_llama.py:633-646,
hashattention_mistral.py:566-594; the trainer writes them with `torch.save(usa_modules.cpu().state_dict(), path)`,
train_hashattention.py:175-178, after `usa_modules.bfloat16()`, :85).

The state dicts are built by hand from the reference's key names
("{layer}.learning_to_hash_transformation_{k,q}.{head}.{0,2,4}.{weight,bias}"; the LSH baseline keeps one projection per
head under three aliased prefixes), written with torch.save and read back through the module API.  Checked: the modules
arrive on the GPU in fp32 holding exactly the file's values (load_state_dict copies into fp32 parameters, whatever the
file's dtype), their codes equal those of modules filled in memory, and - for the learned hashes - those of the oracle
on the raw tensors of the file."""
import types

import pytest
import torch
from torch import nn

from hashattention import hashattention_llama as hl
from hashattention import hashattention_mistral as hm
from hashattention._patched import USA
from oracle import hashattn_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
N_MODEL_LAYERS, N_HEADS, HEAD_DIM = 2, 4, 128


def _config(num_layers, final_dim, with_num_layers=True):
    cfg = types.SimpleNamespace(lth_init_dim=128, lth_final_dim=final_dim, lth_thold=0, num_hidden_layers=N_MODEL_LAYERS,
                                num_attention_heads=N_HEADS, head_dim=HEAD_DIM, hidden_size=N_HEADS * HEAD_DIM)
    if with_num_layers:
        cfg.lth_num_layers = num_layers
    return cfg


def _hand_made_state_dict(num_layers, final_dim, dtype, seed):
    """The tensors a reference checkpoint holds, keyed as nn.ModuleList[USA] names them."""
    g = torch.Generator().manual_seed(seed)
    if num_layers == 0:
        dims, slots = [(HEAD_DIM + 1, final_dim)], [1]          # Sequential(IpToCS(), Linear): the Linear is entry 1
    else:
        dims = {3: [(128, 128), (128, 128), (128, final_dim)], 2: [(128, 128), (128, final_dim)], 1: [(128, final_dim)]}[num_layers]
        slots = [0, 2, 4][:num_layers]
    sd = {}
    for L in range(N_MODEL_LAYERS):
        for h in range(N_HEADS):
            sides = {}
            for side in ("k", "q"):
                if num_layers == 0 and side == "q":
                    sides["q"] = sides["k"]                         # one projection shared by keys and queries
                    continue
                sides[side] = [((torch.randn(fo, fi, generator=g) * fi ** -0.5).to(dtype), (torch.randn(fo, generator=g) * 0.01).to(dtype))
                               for fi, fo in dims]
            for side, layers in sides.items():
                for slot, (w, b) in zip(slots, layers):
                    sd[f"{L}.learning_to_hash_transformation_{side}.{h}.{slot}.weight"] = w
                    sd[f"{L}.learning_to_hash_transformation_{side}.{h}.{slot}.bias"] = b
            if num_layers == 0:
                for slot, (w, b) in zip(slots, sides["k"]):
                    sd[f"{L}.learning_to_hash_transformation.{h}.{slot}.weight"] = w
                    sd[f"{L}.learning_to_hash_transformation.{h}.{slot}.bias"] = b
    return sd


def _heads(sd, L, side, num_layers):
    slots = [1] if num_layers == 0 else [0, 2, 4][:num_layers]
    return [[(sd[f"{L}.learning_to_hash_transformation_{side}.{h}.{s}.weight"].float(),
              sd[f"{L}.learning_to_hash_transformation_{side}.{h}.{s}.bias"].float()) for s in slots] for h in range(N_HEADS)]


CASES = [("llama", 3, 32, torch.float32), ("llama", 3, 32, torch.bfloat16), ("llama", 2, 64, torch.bfloat16),
         ("llama", 0, 32, torch.float32), ("mistral", 3, 32, torch.bfloat16), ("mistral", 3, 32, torch.float32)]


@pytest.mark.parametrize("family,num_layers,final_dim,file_dtype", CASES)
def test_load_usa_from_a_state_dict_file(tmp_path, family, num_layers, final_dim, file_dtype):
    print(f"\n[case] load_usa from file: {family}, {num_layers} layers, {final_dim} bits, {file_dtype}", flush=True)
    api = hl if family == "llama" else hm
    cfg = _config(num_layers, final_dim, with_num_layers=(family == "llama"))      # the Mistral config has no lth_num_layers
    sd = _hand_made_state_dict(num_layers, final_dim, file_dtype, seed=5 + num_layers)
    path = str(tmp_path / "usa.pt")
    torch.save(sd, path)

    usa = api.load_usa(cfg, path)
    assert isinstance(usa, nn.ModuleList) and len(usa) == N_MODEL_LAYERS
    assert all(p.is_cuda and p.dtype == torch.float32 for p in usa.parameters())
    got = usa.state_dict()
    assert set(got) == set(sd)
    for key, t in sd.items():
        assert torch.equal(got[key].cpu(), t.float()), key

    # the same tensors put into modules without a file
    usa_cfg = {"lth_int_dim": 128, "lth_final_dim": final_dim, "lth_thold": 0, "lth_num_layers": num_layers}
    mem = nn.ModuleList([USA(N_HEADS, HEAD_DIM, usa_cfg) for _ in range(N_MODEL_LAYERS)])
    mem.load_state_dict(sd)
    mem = mem.cuda()

    g = torch.Generator().manual_seed(1)
    K = torch.randn(2, N_HEADS, 200, HEAD_DIM, generator=g).to(DEV)
    Q = torch.randn(2, N_HEADS, 3, HEAD_DIM, generator=g).to(DEV)
    for L in range(N_MODEL_LAYERS):
        span, ksign = usa[L](K, Q, hard=True)
        span_m, ksign_m = mem[L](K, Q, hard=True)
        assert torch.equal(span, span_m) and torch.equal(ksign, ksign_m)
        if num_layers > 0:      # learned hashes: the oracle on the file's raw tensors
            span_ref, ksign_ref = orc.usa_forward_hard(K.cpu(), Q.cpu(), _heads(sd, L, "k", num_layers), _heads(sd, L, "q", num_layers))
            assert torch.equal(span.cpu(), span_ref) and torch.equal(ksign.cpu(), ksign_ref)
        else:                   # LSH baseline: keys and queries share the projection, as the three prefixes of the file do
            kmod, qmod = usa[L].learning_to_hash_transformation_k, usa[L].learning_to_hash_transformation_q
            assert all(kmod[h][1].weight is qmod[h][1].weight for h in range(N_HEADS))
            span_ref, ksign_ref = orc.usa_forward_hard(K.cpu(), Q.cpu(), _heads(sd, L, "k", 0), _heads(sd, L, "q", 0), lsh=True)
            assert torch.equal(span.cpu(), span_ref) and torch.equal(ksign.cpu(), ksign_ref)

    # the module turned bf16 (as the trainer keeps it, train_hashattention.py:85): file-loaded and in-memory modules still agree
    usa_b, mem_b = usa.bfloat16(), mem.bfloat16()
    span_b, _ = usa_b[0](K.bfloat16(), Q.bfloat16(), hard=True)
    span_mb, _ = mem_b[0](K.bfloat16(), Q.bfloat16(), hard=True)
    assert torch.equal(span_b, span_mb)


def test_trainer_round_trip_and_layer_count_mismatch(tmp_path):
    # what train_hashattention.py does: modules -> bf16 -> cpu state dict -> torch.save -> load_usa
    print("\n[case] load_usa: trainer round trip", flush=True)
    cfg = _config(3, 32)
    first = hl.load_usa(cfg, None).bfloat16()
    path = str(tmp_path / "ckpt.pt")
    torch.save(first.cpu().state_dict(), path)
    again = hl.load_usa(cfg, path)
    first = first.cuda()
    for (n1, p1), (n2, p2) in zip(first.named_parameters(), again.named_parameters()):
        assert n1 == n2 and p2.dtype == torch.float32 and torch.equal(p1.float(), p2)
    K = torch.randn(1, N_HEADS, 100, HEAD_DIM, device=DEV)
    Q = torch.randn(1, N_HEADS, 1, HEAD_DIM, device=DEV)
    a, _ = first.float()[1](K, Q, hard=True)
    b, _ = again[1](K, Q, hard=True)
    assert torch.equal(a, b)
    # a file for another architecture is refused as torch refuses it (missing / unexpected keys), not half-loaded
    cfg2 = _config(2, 32)
    with pytest.raises(RuntimeError):
        hl.load_usa(cfg2, path)
    # the Mistral API builds three-layer MLPs whatever the config says (its USA has no other form, mistral:77-88)
    cfg3 = _config(2, 32)
    assert all(u.num_layers == 3 for u in hm.load_usa(cfg3, path))
