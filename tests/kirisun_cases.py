"""Shared by the Kirisun tests on the CPU stand-ins and on the GPU: small configurations, model folders whose
weights are made so that a fault shows, and comparisons with the plain implementation (tests/plain_kirisun.py)."""
from __future__ import annotations

import os
import tempfile
from typing import Dict, List

import torch
from safetensors.torch import load_file, save_file

from nano_vllm_amd.config import ChannelDeltaConfig as Delta
from nano_vllm_amd.config import GatedAttentionConfig as Att
from nano_vllm_amd.config import KirisunConfig, KirisunLayer
from nano_vllm_amd.config import SoftmaxExpertsConfig as Moe
from nano_vllm_amd.weights import write_random_model

import plain_kirisun as plain

# Six configurations.  Together: windows smaller and larger than a page and no multiple of it, a window of one
# position, one longer than every prompt and none at all; 0, 1 and several kept first positions, more of them than
# a page and more than the window; two windows in one model (two cache groups); 1, 2 and 3 query heads per
# key/value head; values larger, smaller and as large as keys; rotation of a part of a head, of all of it and none,
# scaling factors of 1 and more; with and without a cap on the scores; delta-rule layers first, last and in a row,
# with 1, 2 and as many query/key heads as value heads, convolutions of 1 to 5 taps, ranks of 1 and more; 1 to 3
# experts a token, layers without a feed-forward; residual multipliers and embedding scales of 1 and other values;
# sizes that are no multiples of 8.
CONFIGS: Dict[str, dict] = {
    "a": dict(cfg=KirisunConfig(vocab=200, width=48, eps=1e-5, residual_mult=0.5, embedding_scale=7.0, layers=(
        KirisunLayer("channel_delta", Delta(heads=4, kv_heads=2, dim=12, vdim=8, conv=3, decay_rank=5, gate_rank=3),
                     Moe(experts=6, top=2, ff=20)),
        KirisunLayer("attention", Att(4, 2, 16, 24, 0.3, softcap=4.0, window=10, keep_first=3, rot_dims=8, rot_base=100.0,
                                      rot_factor=4.0), None),
        KirisunLayer("attention", Att(2, 2, 24, 8, 0.2, softcap=None, window=21, keep_first=0, rot_dims=24, rot_base=1e4,
                                      rot_factor=1.0), Moe(experts=4, top=1, ff=12)),
        KirisunLayer("channel_delta", Delta(heads=2, kv_heads=2, dim=10, vdim=14, conv=1, decay_rank=1, gate_rank=4),
                     Moe(experts=5, top=3, ff=9)))),
        page=8, seed=41),
    # sizes of the matrix-core kernels' kind (multiples of 32 everywhere)
    "b": dict(cfg=KirisunConfig(vocab=512, width=128, eps=1e-6, residual_mult=1.0, embedding_scale=1.0, layers=(
        KirisunLayer("attention", Att(8, 2, 64, 64, 0.11, softcap=30.0, window=48, keep_first=4, rot_dims=32, rot_base=2e5,
                                      rot_factor=3.0), Moe(experts=8, top=3, ff=64)),
        KirisunLayer("channel_delta", Delta(heads=4, kv_heads=2, dim=64, vdim=64, conv=4, decay_rank=16, gate_rank=16),
                     Moe(experts=8, top=3, ff=64)),
        KirisunLayer("attention", Att(8, 2, 64, 64, 0.11, softcap=30.0, window=48, keep_first=4, rot_dims=32, rot_base=2e5,
                                      rot_factor=3.0), Moe(experts=8, top=3, ff=64)))),
        page=32, seed=42),
    "c": dict(cfg=KirisunConfig(vocab=97, width=20, eps=1e-6, residual_mult=0.2, embedding_scale=4.5, layers=(
        KirisunLayer("attention", Att(3, 3, 6, 10, 0.4, softcap=2.0, window=1, keep_first=2), Moe(experts=5, top=3, ff=9)),
        KirisunLayer("channel_delta", Delta(heads=3, kv_heads=1, dim=5, vdim=7, conv=5, decay_rank=2, gate_rank=2), None),
        KirisunLayer("attention", Att(3, 1, 8, 4, 0.5, softcap=9.0, window=4096, keep_first=5, rot_dims=6, rot_base=50.0,
                                      rot_factor=1.5), Moe(experts=9, top=2, ff=6)),
        KirisunLayer("attention", Att(2, 1, 10, 10, 0.35, softcap=None, window=None, rot_dims=10, rot_base=300.0),
                     Moe(experts=3, top=3, ff=8)))),
        page=4, seed=43),
    "d": dict(cfg=KirisunConfig(vocab=333, width=72, eps=1e-6, residual_mult=0.7, embedding_scale=8.5, layers=(
        KirisunLayer("attention", Att(6, 2, 24, 40, 0.25, softcap=6.0, window=5, keep_first=19, rot_dims=24, rot_base=1e6,
                                      rot_factor=8.0), Moe(experts=15, top=2, ff=30)),
        KirisunLayer("channel_delta", Delta(heads=6, kv_heads=3, dim=16, vdim=12, conv=4, decay_rank=4, gate_rank=6),
                     Moe(experts=15, top=2, ff=30)),
        KirisunLayer("channel_delta", Delta(heads=2, kv_heads=1, dim=40, vdim=70, conv=2, decay_rank=3, gate_rank=3), None))),
        page=16, seed=44),
    # a larger one for long prompts: heads of 64 to 128, windows over several pages, a delta-rule head wider than a wave
    "e": dict(cfg=KirisunConfig(vocab=384, width=256, eps=1e-5, residual_mult=0.4, embedding_scale=16.0, layers=(
        KirisunLayer("attention", Att(4, 2, 64, 64, 0.11, softcap=40.0, window=160, keep_first=70, rot_dims=64, rot_base=2e4,
                                      rot_factor=1.0), Moe(experts=10, top=3, ff=72)),
        KirisunLayer("channel_delta", Delta(heads=4, kv_heads=4, dim=96, vdim=80, conv=3, decay_rank=8, gate_rank=8), None),
        KirisunLayer("attention", Att(2, 1, 128, 128, 0.09, softcap=40.0, window=70, keep_first=1, rot_dims=32, rot_base=2e4,
                                      rot_factor=2.0), Moe(experts=10, top=3, ff=72)),
        KirisunLayer("channel_delta", Delta(heads=2, kv_heads=1, dim=128, vdim=128, conv=4, decay_rank=8, gate_rank=8),
                     Moe(experts=10, top=3, ff=72)))),
        page=64, seed=45),
    # ones and equal values: a single head, a single expert, as many kept positions as the window holds, a window of
    # whole pages, multipliers of one, tiny heads
    "f": dict(cfg=KirisunConfig(vocab=50, width=24, eps=1e-6, residual_mult=1.0, embedding_scale=1.0, layers=(
        KirisunLayer("channel_delta", Delta(heads=1, kv_heads=1, dim=8, vdim=8, conv=2, decay_rank=2, gate_rank=2),
                     Moe(experts=1, top=1, ff=8)),
        KirisunLayer("attention", Att(1, 1, 8, 8, 0.35, softcap=None, window=8, keep_first=8, rot_dims=2, rot_base=10.0),
                     Moe(experts=2, top=2, ff=8)),
        KirisunLayer("channel_delta", Delta(heads=2, kv_heads=1, dim=4, vdim=6, conv=4, decay_rank=1, gate_rank=1), None),
        KirisunLayer("attention", Att(2, 1, 4, 4, 0.5, softcap=1.0, window=64, keep_first=64, rot_dims=4, rot_base=1e3,
                                      rot_factor=2.0), None))),
        page=8, seed=46),
}

_folders: Dict[str, str] = {}
_tmp = None


def stretch(tensors: Dict[str, torch.Tensor], seed: int, sharp: bool = True) -> Dict[str, torch.Tensor]:
    """Random weights of N(0, std) hide faults: norms at their neutral values, decays that forget nothing or
    everything at once, router logits that all lie together, gates that all lie at one half.  This makes them
    of a size that shows.  sharp: also peaked softmaxes and router logits far apart, which the float32 tests want
    (a lost key or a wrong expert then moves the logits) and which multiply bfloat16's rounding."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for k, t in tensors.items():
        f = t.float()
        draw = lambda *shape: torch.randn(shape or f.shape, generator=gen)
        if k.endswith("A_log"):
            f = torch.log(0.05 + 1.5 * torch.rand(f.shape, generator=gen))
        elif k.endswith("dt_bias"):
            f = draw() * 1.5 - 1.0
        elif k.endswith(".conv"):
            f = draw() * 0.6
        elif k.endswith(".router"):
            f = draw() * (0.6 if sharp else 0.15)
        elif k.endswith(".router.b"):
            f = draw() * 0.8
        elif k.endswith("norm1") or k.endswith("norm2") or k.endswith("norm1b") or k.endswith("norm2b") or k == "final.norm" \
                or k.endswith(".norm"):
            f = 1.0 + 0.4 * draw()
        elif k.endswith(".a2") or k.endswith(".g2") or k.endswith(".a1") or k.endswith(".g1"):
            f = f * (6.0 if sharp else 3.0)
        elif sharp and (k.endswith(".mix.q") or k.endswith(".mix.k") or k.endswith(".mix.g") or k.endswith(".mix.b")):
            f = f * 3.0                       # peaked softmaxes: a lost key moves the output; gates away from one half
        out[k] = f.to(t.dtype).contiguous()
    return out


def model_folder(name: str, dtype: str = "float32") -> str:
    global _tmp
    key = f"{name}-{dtype}"
    if key not in _folders:
        if _tmp is None:
            _tmp = tempfile.TemporaryDirectory(prefix="nva-kirisun-")
        c = CONFIGS[name]
        path = os.path.join(_tmp.name, key)
        write_random_model(path, c["cfg"], seed=c["seed"], std=0.08, dtype=dtype)
        file = os.path.join(path, "model.safetensors")
        save_file(stretch(load_file(file), c["seed"], sharp=dtype == "float32"), file, metadata={"format": "pt"})
        _folders[key] = path
    return _folders[key]


_plain_cache: Dict[str, tuple] = {}


def plain_model(folder: str):
    if folder not in _plain_cache:
        _plain_cache[folder] = plain.read_folder(folder, torch.float64)
    return _plain_cache[folder]


def plain_logits(folder: str, tokens: List[int]) -> torch.Tensor:
    cfg, w = plain_model(folder)
    return plain.forward(cfg, w, list(tokens)).float()


def errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per position: the difference of the logits (their mean taken off), root mean square over the
    vocabulary, against the spread of the wanted logits."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    spread = want.double() - want.double().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / spread.pow(2).mean().sqrt()


def err(got: torch.Tensor, want: torch.Tensor) -> float:
    return float(errors(got, want).max())
