"""Small Vuzazen configurations for tests, and the maker of their model folders.

A: every mixer type in the order memory, attention, latent, attention; 2 of 4 experts and a dense feed-forward; a layer
   without feed-forward; 3 query heads a kv head; 3 taps and an attention layer without a convolution; value heads wider
   than key heads in the attention and in the memory.
B: the values another model may make equal or 1: as many kv heads as heads, one memory head, one expert of two chosen
   and all experts chosen, 2 taps, value size = key size, a width that is no multiple of 8, a latent layer first, an
   embedding scale of 1, a bucket count of 1.
C: one kv head, 5 taps, sizes in no kernel's favourite multiples (width 50, heads of 12 and 20), memories only behind the
   first layer, a query latent wider than the key latent, large multipliers of the pair table.
M: memories alone (no layer keeps pages): requests have states and lengths, and no cache to read.
R: real-looking head sizes (64 and 128, a latent of 112 + 16, memories of 64 by 96 and 128 by 64) with pages of 64, for the
   matrix-core kernels; mixed heads over two kv heads of 128 (one key head of 256).
S: the matrix-core kernels' sizes again: three kv heads of 32 with values of 128 and four query heads each (single
   tokens then take a group's heads as the rows of a block), four kv heads of 64 that are all the heads, 4 taps and one tap, 3 of 8
   experts.

Random routers would leave some token's choice of experts to a difference that bfloat16 does not keep: `make_model`
writes weights in which the choice is decided by a few columns of the stream that only the embedding writes to (the
last MARKERS columns hold +-MARK by the bits of the token's id; the pair table and every product that adds to the stream
have zeros there; the routers read those columns alone; a norm scales them all alike, which keeps the order of the
logits).  A memory's answer is S^T q divided by |n . q| where that is above its floor, and bfloat16 does not keep the
sign or the size of an n . q near zero: one more column of the stream holds the same number for every token, and the
memories' queries and keys both read it strongly, so that q . k is clearly positive for every pair of tokens and n . q
stays away from zero (the tests' keys also lean towards their queries).
"""
import os

import torch

MARKERS = 3
MARK = 2.0
MARGIN = 0.1         # least distance between the last chosen logit and the first left out, markers taken as +-1


def _mem(heads, dim, vdim, cap, mlp):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": mlp}


def _lat(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base, mlp):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
                                                  "q_rank": q_rank, "scale": scale, "rot": {"dims": rot_dim, "base": base}},
            "mlp": mlp}


def _att(heads, kv_heads, dim, vdim, scale, conv, mlp):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if conv:
        m["conv"] = conv
    return {"type": "attention", "mixer": m, "mlp": mlp}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def _config(vocab, width, eps, scale, bigram, layers):
    return {"architecture": "Vuzazen", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": scale, "bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))}, "layers": layers}


MODELS = {
    "A": dict(config=_config(311, 96, 1e-5, 4.0, (97, 31, 5), [
        _mem(3, 16, 24, 8.0, _moe(40, 4, 2)),
        _att(6, 2, 16, 24, 0.4, 3, _dense(160)),
        _lat(4, 16, 8, 24, 40, 24, 0.3, 10000.0, None),
        _att(4, 2, 8, 16, 0.5, 0, _moe(32, 5, 1))]),
        seed=31, linear_std=0.08, norm_std=0.1, page_size=16),
    "B": dict(config=_config(257, 100, 1e-6, 1.0, (1, 3, 1), [
        _lat(2, 24, 4, 24, 24, 24, 0.25, 100.0, _moe(24, 2, 1)),
        _att(5, 5, 20, 20, 0.35, 2, _moe(16, 3, 3)),
        _mem(1, 20, 20, 15.0, _dense(72))]),
        seed=32, linear_std=0.1, norm_std=0.2, page_size=8),
    "C": dict(config=_config(131, 50, 1e-5, 2.5, (30, 1000003, 99991), [
        _att(3, 1, 12, 20, 0.5, 5, _dense(34)),
        _mem(2, 20, 12, 4.0, None),
        _lat(3, 12, 6, 10, 18, 26, 0.3, 50.0, _moe(18, 6, 4)),
        _mem(5, 6, 10, 30.0, _dense(40))]),
        seed=33, linear_std=0.1, norm_std=0.1, page_size=8),
    "M": dict(config=_config(190, 72, 1e-6, 8.0, (64, 5, 9), [
        _mem(2, 24, 32, 10.0, _dense(48)),
        _mem(4, 8, 8, 6.0, _moe(24, 4, 2))]),
        seed=34, linear_std=0.1, norm_std=0.15, page_size=8),
    "R": dict(config=_config(409, 384, 1e-6, 12.0, (2039, 211, 19), [
        _lat(6, 64, 16, 48, 112, 72, 0.1, 10000.0, _dense(768)),
        _mem(3, 64, 96, 11.0, _moe(128, 8, 2)),
        _att(4, 2, 128, 64, 0.09, 3, _dense(512)),
        _mem(2, 128, 64, 9.0, None)]),
        seed=35, linear_std=0.04, norm_std=0.1, page_size=64),
    "S": dict(config=_config(300, 320, 1e-5, 10.0, (601, 17, 129), [
        _att(12, 3, 32, 128, 0.18, 4, _moe(64, 8, 3)),
        _att(4, 4, 64, 64, 0.12, 1, _dense(320)),
        _lat(5, 48, 32, 64, 80, 56, 0.14, 500000.0, None)]),
        seed=36, linear_std=0.05, norm_std=0.1, page_size=64),
}


def make_model(model_dir, name):
    """Writes the folder of configuration `name` (random weights, decisive routers, keys that lean towards their
    queries in the memories); returns the folder."""
    from safetensors import safe_open
    from safetensors.torch import save_file
    from xinfer_amd.weights import write_random_model
    t = MODELS[name]
    write_random_model(model_dir, t["config"], t["seed"], t["linear_std"], t["norm_std"])
    path = os.path.join(model_dir, "model.safetensors")
    W = {}
    with safe_open(path, framework="pt") as f:
        for k in f.keys():
            W[k] = f.get_tensor(k).clone()
    c = t["config"]
    width = c["width"]
    cols = list(range(width - MARKERS, width))
    same = width - MARKERS - 1                              # the column that is the same for every token
    ids = torch.arange(c["vocab"])
    W["embed"][:, same] = MARK / c["embedding"]["scale"]
    W["bigram"][:, same] = 0
    for b, col in enumerate(cols):
        W["embed"][:, col] = (((ids >> b) & 1).float() * 2 - 1) * MARK / c["embedding"]["scale"]
    W["bigram"][:, cols] = 0
    g = torch.Generator().manual_seed(t["seed"])
    for name_, w in W.items():
        if name_.endswith((".mix.o", ".down")):             # nothing but the embedding writes to the marker columns
            w[cols + [same], :] = 0
    for i, layer in enumerate(c["layers"]):
        if layer["type"] == "mlstm":
            W[f"l{i}.mix.k"] = (W[f"l{i}.mix.q"].float() + 0.5 * W[f"l{i}.mix.k"].float()).to(torch.bfloat16)
            W[f"l{i}.norm1"][same] = 0.0
            for part in ("q", "k"):
                W[f"l{i}.mix.{part}"][:, same] = 0.5
            for gate in ("i", "f"):                         # gates that move with the token, up to their cap
                W[f"l{i}.mix.{gate}"] = (W[f"l{i}.mix.{gate}"].float() * 6).to(torch.bfloat16)
        ml = layer.get("mlp")
        if not ml or ml["kind"] != "moe":
            continue
        W[f"l{i}.norm2"][cols] = 0.0                        # a factor of 1
        top, experts = ml["router"]["top"], ml["router"]["experts"]
        pats = torch.tensor([[1.0 if (p >> b) & 1 else -1.0 for b in range(MARKERS)] for p in range(1 << MARKERS)])
        for _ in range(20000):            # until every pattern's choice is clear by MARGIN
            rw = (torch.randn(experts, MARKERS, generator=g) * 0.5).to(torch.bfloat16).float()
            z = (pats @ rw.T).sort(dim=-1, descending=True).values
            if top == experts or float((z[:, top - 1] - z[:, top]).min()) >= MARGIN:
                break
        else:
            raise RuntimeError("no decisive router found")
        r = torch.zeros_like(W[f"l{i}.mlp.router"], dtype=torch.float32)
        r[:, cols] = rw
        W[f"l{i}.mlp.router"] = r.to(torch.bfloat16)
    save_file({k: v.contiguous() for k, v in W.items()}, path)
    return model_dir
