"""Small Lagedra configurations and weights for the tests: sizes that differ from layer to
layer and between the configurations (one to six heads, grouped and ungrouped key/value heads,
key and value sizes on either side of each other and off the multiples of 8, whole and partial
rotation with and without stretched frequencies, windows of 1, of a page and wider than the
prompts, one to five taps, decays from fast to none, experts in one group or several with one
or more kept, one to four experts chosen, layers without a feed-forward, either kind of layer
first, models with one kind of layer only), and weights at scales at which every mechanism
matters: norm weights, head temperatures, value mixes and depth weights spread out, scores
that reach the cap."""
from __future__ import annotations

from typing import Dict, List

import torch

from bekunex_models import judge  # noqa: F401
from gipotar_models import (as_stored, prompts, row_error, write_folder,  # noqa: F401
                            TOLERANCE)


def _moe(ff, limit, experts, groups, keep, top):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "groups": {"count": groups, "keep": keep}, "top": top}}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _lightning(heads, dim, vdim, decay, mlp):
    return {"type": "lightning", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}}


def _attention(heads, kv_heads, dim, vdim, conv, window, rot_dims, base, scaling, scale, softcap,
               v_mix, mlp):
    rot = {"base": base, "dims": rot_dims}
    if scaling is not None:
        factor, original, fast, slow = scaling
        rot["scaling"] = {"factor": factor, "original": original, "fast": fast, "slow": slow}
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
                      "mask": {"size": window}, "rot": rot, "scale": scale, "softcap": softcap,
                      "v_mix": v_mix}}


# Both kinds of layer, attention first; three value-mixing layers of which the first is not the
# first attention layer; partial rotation; a window shorter than two pages and one of a page.
CONFIG_A = {
    "architecture": "Lagedra", "vocab": 97, "width": 48, "max_positions": 512,
    "norm": {"eps": 1e-5},
    "layers": [
        _attention(4, 2, 16, 24, 3, 20, 8, 1000.0, (4.0, 64, 8.0, 1.0), 0.3, 6.0, False,
                   _dense(72)),
        _lightning(3, 24, 40, [0.5, 0.9, 0.999], _moe(24, 1.5, 6, 3, 2, 2)),
        _attention(6, 2, 8, 12, 2, 16, 8, 40000.0, None, 0.4, 4.0, True, None),
        _lightning(2, 16, 8, [1.0, 0.7], _dense(40)),
        _attention(2, 2, 24, 12, 4, 33, 16, 300.0, (2.0, 32, 4.0, 0.5), 0.25, 9.0, True,
                   _moe(16, 0.7, 4, 1, 1, 1)),
        _attention(1, 2, 12, 12, 1, 200, 12, 10000.0, (8.0, 128, 32.0, 1.0), 0.3, 5.0, True,
                   _moe(20, 2.0, 8, 4, 3, 4)),
    ],
}
CONFIG_A["layers"][5]["mixer"]["heads"] = 2
# Only linear attention (no mixer asks for pages), sizes off every multiple of 4.
CONFIG_B = {
    "architecture": "Lagedra", "vocab": 64, "width": 40, "max_positions": 400,
    "norm": {"eps": 1e-6},
    "layers": [
        _lightning(5, 6, 10, [0.3, 0.6, 0.9, 0.99, 0.9995], _moe(12, 1.0, 5, 1, 1, 2)),
        _lightning(1, 70, 33, [0.97], None),
        _lightning(2, 130, 16, [0.8, 0.95], _dense(56)),
    ],
}
# Only attention; head sizes and rotated widths off the multiples of 8, a window of one
# position, one tap (no state at all), key/value heads of one, every query head its own.
CONFIG_C = {
    "architecture": "Lagedra", "vocab": 80, "width": 56, "max_positions": 300,
    "norm": {"eps": 1e-6},
    "layers": [
        _attention(3, 3, 12, 20, 5, 16, 6, 300.0, None, 0.28, 7.0, True, _moe(20, 1.2, 4, 2, 2, 2)),
        _attention(4, 1, 10, 10, 1, 1, 10, 1000.0, (3.0, 40, 6.0, 2.0), 0.3, 3.0, False, None),
        _attention(6, 3, 20, 20, 2, 47, 4, 20000.0, (16.0, 16, 2.0, 1.0), 0.22, 8.0, True,
                   _dense(30)),
    ],
}
# Head sizes that the matrix-core kernels take as they are (64 with the whole head rotated, which
# the attention kernels can do themselves; 128 and 32 for keys and values with half the head
# rotated; 48 and 64, padded to one size), heads of 64 and 128 channels in the linear attention,
# for prompts of hundreds of tokens.
CONFIG_D = {
    "architecture": "Lagedra", "vocab": 200, "width": 128, "max_positions": 1024,
    "norm": {"eps": 1e-6},
    "layers": [
        _lightning(2, 64, 64, [0.9, 0.995], _dense(192)),
        _attention(4, 2, 64, 64, 3, 100, 64, 10000.0, (8.0, 256, 16.0, 2.0), 0.125, 15.0, True,
                   _moe(64, 1.0, 8, 2, 1, 2)),
        _lightning(1, 128, 128, [0.98], _moe(32, 2.0, 4, 2, 2, 3)),
        _attention(2, 1, 128, 32, 4, 40, 64, 500000.0, None, 0.09, 25.0, False, _dense(160)),
        _attention(4, 2, 48, 64, 2, 300, 48, 20000.0, (2.0, 512, 8.0, 1.0), 0.14, 10.0, True, None),
    ],
}
# A width, feed-forward widths and a vocabulary that are no multiples of 8 (rows that do not
# start on 16-byte boundaries in bfloat16), one head.  Every expert is chosen: behind a choice
# that bfloat16 rounding can flip, the head that forgets nothing would carry the other expert's
# output through all later rows.
CONFIG_E = {
    "architecture": "Lagedra", "vocab": 333, "width": 100, "max_positions": 260,
    "norm": {"eps": 1e-5},
    "layers": [
        _lightning(1, 36, 52, [0.93], _moe(30, 1.0, 3, 1, 1, 3)),
        _attention(1, 1, 28, 36, 3, 24, 14, 5000.0, (4.0, 48, 4.0, 1.0), 0.2, 12.0, True,
                   _dense(150)),
        _attention(3, 1, 20, 36, 2, 60, 20, 900.0, None, 0.22, 6.0, True, _moe(25, 3.0, 6, 2, 2, 6)),
        _lightning(5, 20, 12, [0.6, 0.8, 0.9, 0.95, 1.0], _dense(70)),
    ],
}
CONFIGS = {"a": CONFIG_A, "b": CONFIG_B, "c": CONFIG_C, "d": CONFIG_D, "e": CONFIG_E}


def spec_of(config: dict):
    from rust_llm_inference_server_amd.registry import architecture_of
    arch = architecture_of(config)
    return arch.build_spec(arch.parse_config(config))


def make_weights(config: dict, seed: int) -> Dict[str, torch.Tensor]:
    """float32 tensors by checkpoint name, values chosen by what the tensor is."""
    g = torch.Generator().manual_seed(seed)
    normal = lambda shape, std=1.0: torch.randn(shape, generator=g) * std
    uniform = lambda shape, lo, hi: lo + (hi - lo) * torch.rand(shape, generator=g)
    out = {}
    for t in spec_of(config).tensor_specs():
        name, shape = t.name, tuple(t.shape)
        last = name.split(".")[-1]
        if name == "embed":
            w = normal(shape, 0.5)
        elif name == "pos":
            w = normal(shape, 0.3)
        elif last in ("norm1", "norm2") or name == "final.norm":
            w = 1.0 + normal(shape, 0.3)
        elif last == "norm":
            w = 1.0 + normal(shape, 0.3)
        elif last == "dwa":
            w = 1.0 / shape[0] + normal(shape, 0.3)
        elif last == "temp":
            w = uniform(shape, 0.5, 1.8)
        elif last == "vmix":
            w = uniform(shape, 0.2, 0.8)
        elif last == "conv":
            w = normal(shape, 0.6)
        elif last == "router":
            w = normal(shape, 2.0 * shape[1] ** -0.5)
        elif len(shape) == 2:
            w = normal(shape, shape[1] ** -0.5)
        else:
            raise AssertionError(f"no rule for {name}")
        out[name] = w.contiguous()
    return out


def plain_logits(plain, cfg: dict, stored: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    return plain.forward(cfg, stored, tokens)[0]
