"""The tests' own small Barotar configurations; they differ in every size, constant and option: the order of the
layers, layers without a feed-forward, values of another size than the keys, heads that are no multiple of anything,
rotations of a part of a head, of the whole head and of nothing, windows from one key to more than any test feeds,
one and several key/value heads, inner sizes of the decays from 1 up, one group of experts and one expert a group, all
groups kept, one expert chosen and several, more heads than an attention tile holds."""
from __future__ import annotations

import functools
import tempfile

import plain_barotar as plain
from llmserver_amd.config import config_from_dict
from llmserver_amd.weights import RandomInit, write_random_model


def attention(heads, kv_heads, dim, vdim, window, rot_dims, base=10000.0, scale=None, softcap=30.0):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window}, "rot": {"base": base, "dims": rot_dims},
            "scale": scale if scale is not None else dim ** -0.5, "softcap": softcap}


def parallel(left, heads, dim, low=None, left_scale=1.0, right_scale=1.0):
    right = {"heads": heads, "dim": dim}
    if low is not None:
        right["low"] = low
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}}


def gla(heads, dim, vdim, tau, low=None):
    mixer = {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}
    if low is not None:
        mixer["low"] = low
    return {"type": "gla", "mixer": mixer}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, limit, experts, top, groups, keep):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}


def config(vocab, width, eps, layers):
    return {"architecture": "Barotar", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "layers": [{**mixer, "mlp": mlp} for mixer, mlp in layers]}


BA = config(97, 48, 1e-5, [
    (parallel(attention(4, 2, 12, 20, 7, 4, base=100.0, scale=0.3, softcap=5.0), 3, 10, low=5, left_scale=0.7, right_scale=1.2), dense(40)),
    (gla(2, 6, 9, 3.0, low=3), moe(12, 0.8, 6, 2, 3, 2)),
    (parallel(attention(6, 3, 8, 8, 33, 8, base=50.0, softcap=2.0), 2, 24, left_scale=1.1, right_scale=0.6), moe(10, 1.5, 8, 3, 2, 1))])
BB = config(130, 64, 1e-6, [
    (gla(3, 16, 20, 16.0), dense(70)),
    (gla(1, 40, 7, 1.0, low=1), None),
    (parallel(attention(3, 3, 16, 16, 500, 16, base=1e6, scale=0.2, softcap=50.0), 4, 16, low=7), moe(24, 2.0, 4, 1, 4, 4)),
    (gla(5, 4, 12, 8.0, low=9), moe(9, 0.5, 5, 5, 1, 1))])
BC = config(61, 40, 3e-4, [
    (parallel(attention(17, 1, 6, 10, 1, 0, softcap=1.0), 1, 40, low=2, left_scale=-0.5, right_scale=1.0), None),
    (parallel(attention(2, 2, 24, 4, 20, 6, base=77.0, scale=0.4, softcap=8.0), 5, 8, left_scale=1.0, right_scale=0.0), dense(33)),
    (parallel(attention(8, 4, 10, 10, 64, 10, base=300.0), 3, 12, low=20), moe(7, 1.0, 9, 2, 9, 3))])
# Sizes in the kernels' own steps (heads of 32, pages of 16): the padded rows have nothing to pad.
BD = config(200, 64, 1e-5, [
    (parallel(attention(4, 2, 32, 32, 40, 16, base=2e4, scale=0.18, softcap=20.0), 2, 32, left_scale=0.9, right_scale=0.8), moe(32, 1.2, 8, 2, 4, 2)),
    (gla(2, 32, 32, 12.0), dense(96))])
BE = config(50, 32, 1e-5, [(gla(2, 8, 8, 2.0, low=4), moe(8, 1.0, 2, 2, 2, 2))])

INIT = RandomInit(seed=3, std=0.15, norm_noise=0.3, bias_std=0.4)
CASES = {"BA": (BA, INIT, 16), "BB": (BB, RandomInit(seed=8, std=0.12, norm_noise=0.2, bias_std=0.5), 8),
         "BC": (BC, RandomInit(seed=21, std=0.2, norm_noise=0.25, bias_std=0.3), 4), "BD": (BD, INIT, 16),
         "BE": (BE, RandomInit(seed=2, std=0.25, norm_noise=0.3, bias_std=0.6), 8)}

_FOLDERS = {}


def model_folder(case: str) -> str:
    if case not in _FOLDERS:
        raw, init, _ = CASES[case]
        folder = tempfile.mkdtemp(prefix=f"llmserver_amd_test_{case}_")
        write_random_model(config_from_dict(dict(raw)), folder, init)
        _FOLDERS[case] = folder
    return _FOLDERS[case]


@functools.lru_cache(maxsize=None)
def plain_model(case: str):
    return plain.read_folder(model_folder(case))


@functools.lru_cache(maxsize=None)
def plain_logits(case: str, tokens: tuple):
    raw, tensors = plain_model(case)
    return plain.forward(raw, tensors, list(tokens))
