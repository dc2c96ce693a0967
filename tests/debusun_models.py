"""Small Debusun configurations for tests, and the maker of their model folders.

A: every mixer type; the span 1..3 runs twice; attention with value heads wider than its key heads, groups of 3 query
   heads, half of a head rotated (the head-at-a-time kernels) and attention with equal sizes and whole heads rotated (the
   plain form's kernels); a state space with 2 groups, 2 norm groups and 3 taps; a layer without feed-forward; three
   windows (three cache groups).
B: the values other models happen to make equal or 1: the span is the whole model (it starts at layer 0 and nothing
   follows it) and runs three times; as many kv heads as heads; as many groups and norm groups as heads; 2 taps; a window
   of 5; value heads narrower than key heads; a width that is no multiple of 8.
C: no span at all; the state space first, 5 taps, one group; a window of 1 and windows wider than any request; one kv
   head; sizes in no kernel's favourite multiples (width 50, heads of 12 and 20).
D: a span that runs once (its table has one row); a latent layer last; a window of 2.
R: real-looking head sizes (64 and 128, a latent of 128 + 32) with pages of 64, for the matrix-core kernels.
S: the matrix-core kernels' sizes again with what R leaves out: equal key and value head sizes of which only a part
   turns (half of 64, a quarter of 128), a latent of 64 + 16 for 6 heads with values wider than the plain key dims, a
   state space with 3 groups and states of 32; the span is the state space and the latent, twice (a latent on the
   matrix cores with a cache a pass).
"""
import os

import torch


def _rot(dims, base, scaling=None):
    r = {"dims": dims, "base": base}
    if scaling:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


def _att(heads, kv_heads, dim, vdim, scale, window, rot, ff):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                                           "mask": {"size": window}, "rot": rot},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _lat(heads, dim, rot_dim, vdim, rank, scale, window, rot, ff):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
                                                  "scale": scale, "mask": {"size": window}, "rot": rot},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _ssm(heads, vdim, state, groups, conv, norm_groups, ff):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _config(vocab, width, eps, scale, bigram, layers, loop=None):
    c = {"architecture": "Debusun", "vocab": vocab, "width": width, "norm": {"eps": eps},
         "embedding": {"scale": scale, "bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))}, "layers": layers}
    if loop:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    return c


MODELS = {
    "A": dict(config=_config(311, 96, 1e-5, 4.0, (97, 31, 7), [
        _ssm(4, 24, 16, 2, 3, 2, 160),
        _att(6, 2, 16, 24, 0.4, 12, _rot(8, 10000.0), None),
        _lat(4, 16, 8, 24, 40, 0.3, 21, _rot(8, 10000.0, (4.0, 16, 8.0, 1.0)), 128),
        _att(4, 4, 32, 32, 0.25, 30, _rot(32, 500.0), 96)], loop=(1, 3, 2)),
        seed=21, linear_std=0.08, norm_std=0.1, page_size=16),
    "B": dict(config=_config(257, 100, 1e-6, 1.0, (53, 3, 1), [
        _lat(2, 24, 4, 16, 24, 0.25, 9, _rot(4, 100.0, (2.0, 8, 4.0, 0.5)), 72),
        _ssm(3, 20, 8, 3, 2, 3, None),
        _att(5, 5, 20, 12, 0.35, 5, _rot(20, 10000.0), 56)], loop=(0, 3, 3)),
        seed=22, linear_std=0.1, norm_std=0.2, page_size=8),
    "C": dict(config=_config(131, 50, 1e-5, 2.5, (30, 11, 13), [
        _ssm(2, 20, 12, 1, 5, 1, 34),
        _att(3, 1, 12, 20, 0.5, 1, _rot(6, 100.0), 18),
        _lat(3, 12, 6, 10, 18, 0.3, 200, _rot(6, 50.0, (8.0, 32, 16.0, 2.0)), None),
        _att(2, 1, 20, 20, 0.3, 300, _rot(10, 1000.0), 40)]),
        seed=23, linear_std=0.1, norm_std=0.1, page_size=8),
    "D": dict(config=_config(190, 72, 1e-6, 8.0, (64, 5, 9), [
        _att(3, 3, 24, 24, 0.3, 2, _rot(24, 10000.0), 40),
        _ssm(6, 12, 16, 3, 4, 1, 64),
        _lat(6, 8, 2, 8, 16, 0.4, 17, _rot(2, 10000.0, (3.0, 10, 2.0, 1.0)), 48)], loop=(1, 2, 1)),
        seed=24, linear_std=0.1, norm_std=0.15, page_size=8),
    "R": dict(config=_config(409, 512, 1e-6, 12.0, (2039, 211, 19), [
        _lat(8, 64, 32, 64, 128, 0.1, 150, _rot(32, 10000.0, (8.0, 64, 32.0, 1.0)), 768),
        _att(8, 2, 64, 128, 0.125, 100, _rot(32, 500000.0), 512),
        _ssm(8, 64, 64, 1, 4, 1, 512),
        _att(4, 4, 128, 128, 0.09, 300, _rot(128, 500000.0), 512)], loop=(1, 4, 2)),
        seed=25, linear_std=0.04, norm_std=0.1, page_size=64),
    "S": dict(config=_config(300, 384, 1e-5, 10.0, (509, 17, 129), [
        _att(4, 2, 64, 64, 0.125, 70, _rot(32, 10000.0), 256),
        _att(2, 1, 128, 128, 0.09, 200, _rot(32, 500000.0), None),
        _ssm(6, 32, 32, 3, 4, 2, 320),
        _lat(6, 32, 16, 48, 64, 0.14, 90, _rot(16, 10000.0, (4.0, 128, 16.0, 2.0)), 256)], loop=(2, 4, 2)),
        seed=26, linear_std=0.05, norm_std=0.1, page_size=64),
}


def make_model(model_dir, name):
    """Writes the folder of configuration `name` (random weights); returns the folder."""
    from xinfer_amd.weights import write_random_model
    t = MODELS[name]
    return write_random_model(model_dir, t["config"], t["seed"], t["linear_std"], t["norm_std"])
