"""The tests' own small Zepolix configurations; they differ in every size, constant and option (layers of unequal
sizes, a layer without a feed-forward, one expert chosen or all, a rotation of a part of the rotated dimensions, a
convolution of two to five taps or none, more heads than an attention tile holds)."""
from __future__ import annotations

import functools
import tempfile

import plain_zepolix as plain
from llmserver_amd.config import config_from_dict
from llmserver_amd.weights import RandomInit, write_random_model


def mixer(heads, dim, rot_dim, vdim, kv_rank, base=10000.0, dims=None, scale=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
            "scale": scale if scale is not None else (dim + rot_dim) ** -0.5, "rot": {"base": base, "dims": dims or rot_dim}}


def experts(ff, count, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": count, "top": top}}


def layer(mix, mlp):
    return {"type": "latent_attention", "mixer": mix, "mlp": mlp}


def config(vocab, width, eps, taps, layers):
    raw = {"architecture": "Zepolix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if taps:
        raw["canon"] = {"taps": taps}
    return raw


ZA = config(97, 48, 1e-5, 3, [layer(mixer(3, 8, 4, 6, 20), experts(12, 5, 2)) for _ in range(3)])
ZB = config(130, 64, 1e-6, 4, [layer(mixer(5, 12, 8, 10, 40, base=500.0, dims=4), experts(20, 3, 1)),
                               layer(mixer(2, 16, 2, 24, 14, base=1e6, scale=0.31), None),
                               layer(mixer(4, 6, 6, 5, 30, base=77.0), experts(9, 4, 4))])
ZC = config(61, 40, 3e-4, 0, [layer(mixer(17, 4, 2, 3, 12), experts(7, 9, 3)), layer(mixer(1, 24, 8, 40, 24), experts(16, 2, 1))])
ZD = config(200, 72, 1e-5, 2, [layer(mixer(6, 10, 6, 12, 58, base=2e4), experts(24, 6, 2)) for _ in range(2)])
ZE = config(50, 32, 1e-5, 5, [layer(mixer(2, 8, 8, 8, 8, base=100.0), experts(8, 2, 2))])
# Two layers with the same number of heads whose cache rows differ in width (two groups of pages, two attention plans), the
# second as wide as the kernels' widest head with the smaller tile shape.
ZF = config(77, 56, 2e-5, 3, [layer(mixer(4, 8, 4, 8, 24), experts(16, 4, 2)), layer(mixer(4, 12, 10, 6, 130, base=3000.0), experts(8, 3, 1))])

INIT = RandomInit(seed=3, std=0.15, norm_noise=0.3, bias_std=0.2)
CASES = {"ZA": (ZA, INIT, 16), "ZB": (ZB, RandomInit(seed=8, std=0.12, norm_noise=0.2, bias_std=0.3), 8),
         "ZC": (ZC, RandomInit(seed=21, std=0.2, norm_noise=0.25, bias_std=0.1), 4), "ZD": (ZD, INIT, 16),
         "ZE": (ZE, RandomInit(seed=2, std=0.25, norm_noise=0.3, bias_std=0.2), 8),
         "ZF": (ZF, RandomInit(seed=13, std=0.12, norm_noise=0.2, bias_std=0.2), 16)}

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
