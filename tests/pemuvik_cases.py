"""Shared by the Pemuvik tests on the CPU stand-ins and on the GPU: small configurations, model folders whose
weights are made so that a fault shows, a paged batch for the attention kernels, and comparisons with the plain
implementation (tests/plain_pemuvik.py)."""
from __future__ import annotations

import os
import random
import tempfile
from types import SimpleNamespace
from typing import Dict, List

import torch
from safetensors.torch import load_file, save_file

from nano_vllm_amd.config import ChoiceExpertsConfig as Moe
from nano_vllm_amd.config import LatentAttentionConfig as Lat
from nano_vllm_amd.config import PemuvikConfig, PemuvikLayer
from nano_vllm_amd.config import SigmoidAttentionConfig as Att
from nano_vllm_amd.weights import write_random_model

import plain_pemuvik as plain

# Five configurations.  Together: windows smaller and larger than a page and no multiple of it, a window of one
# position, one longer than every prompt and none at all; 1, 2 and 3 query heads per key/value head; values larger,
# smaller and as large as keys; rotation of a part of a head, of all of it and none; layers that mix values and
# layers that do not, the first mixing layer first and behind other layers; latent layers first, last and in a row,
# latents smaller and larger than the heads' keys, key rows of up to 128 entries and beyond; dense layers, routed
# ones with and without identities, groups, a shared expert, one expert, as many chosen as there are; layers
# without a feed-forward; sizes that are no multiples of 8.
CONFIGS: Dict[str, dict] = {
    "a": dict(cfg=PemuvikConfig(vocab=200, width=48, eps=1e-5, layers=(
        PemuvikLayer("attention", Att(4, 2, 16, 24, 0.3, window=10, rot_dims=8, rot_base=100.0, v_mix=True), 40),
        PemuvikLayer("attention", Att(2, 2, 12, 24, 0.25, window=21, rot_dims=12, rot_base=1e4, v_mix=True),
                     Moe(experts=6, top=3, ff=20, identity=2, group_count=4, group_keep=2, shared_ff=16)),
        PemuvikLayer("latent_attention", Lat(heads=3, dim=10, rot_dim=6, vdim=14, kv_rank=20, scale=0.3, rot_base=50.0), 24),
        PemuvikLayer("attention", Att(3, 1, 8, 8, 0.4, window=7, rot_dims=0, v_mix=False), Moe(experts=5, top=2, ff=12)),
        PemuvikLayer("attention", Att(4, 2, 8, 24, 0.35, window=33, rot_dims=4, rot_base=1e3, v_mix=True), None),
        PemuvikLayer("latent_attention", Lat(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=12, scale=0.25, rot_base=1e4), None))),
        page=8, seed=51),
    # sizes of the matrix cores' kind (multiples of 32 everywhere)
    "b": dict(cfg=PemuvikConfig(vocab=512, width=128, eps=1e-6, layers=(
        PemuvikLayer("attention", Att(8, 2, 64, 64, 0.11, window=48, rot_dims=32, rot_base=2e5, v_mix=True),
                     Moe(experts=8, top=3, ff=64, identity=0, group_count=2, group_keep=1, shared_ff=64)),
        PemuvikLayer("latent_attention", Lat(heads=4, dim=32, rot_dim=32, vdim=32, kv_rank=64, scale=0.12, rot_base=1e4), 192),
        PemuvikLayer("attention", Att(8, 2, 64, 64, 0.11, window=48, rot_dims=32, rot_base=2e5, v_mix=True),
                     Moe(experts=8, top=3, ff=64, identity=4, group_count=3, group_keep=2, shared_ff=None)))),
        page=32, seed=52),
    # ones and equal values: a latent layer first, one head, one expert, as many chosen as there are, a window of
    # one position and one longer than every request, no mask at all, tiny heads
    "c": dict(cfg=PemuvikConfig(vocab=97, width=20, eps=1e-6, layers=(
        PemuvikLayer("latent_attention", Lat(heads=1, dim=4, rot_dim=2, vdim=6, kv_rank=5, scale=0.5, rot_base=10.0),
                     Moe(experts=1, top=1, ff=8)),
        PemuvikLayer("attention", Att(1, 1, 6, 10, 0.4, window=1, rot_dims=6, rot_base=50.0, v_mix=True),
                     Moe(experts=2, top=3, ff=6, identity=1)),
        PemuvikLayer("attention", Att(3, 1, 8, 10, 0.5, window=4096, rot_dims=2, rot_base=300.0, v_mix=True), 9),
        PemuvikLayer("attention", Att(2, 1, 10, 10, 0.35, window=None, rot_dims=10, rot_base=300.0, v_mix=True),
                     Moe(experts=3, top=3, ff=8, identity=0, shared_ff=5)))),
        page=4, seed=53),
    "d": dict(cfg=PemuvikConfig(vocab=333, width=72, eps=1e-6, layers=(
        PemuvikLayer("latent_attention", Lat(heads=6, dim=12, rot_dim=8, vdim=10, kv_rank=40, scale=0.22, rot_base=1e6), 100),
        PemuvikLayer("latent_attention", Lat(heads=2, dim=24, rot_dim=16, vdim=40, kv_rank=16, scale=0.15, rot_base=500.0),
                     Moe(experts=13, top=2, ff=30, identity=2, group_count=5, group_keep=3, shared_ff=20)),
        PemuvikLayer("attention", Att(6, 3, 24, 16, 0.25, window=5, rot_dims=24, rot_base=1e6, v_mix=False), 50),
        PemuvikLayer("attention", Att(6, 2, 16, 40, 0.3, window=19, rot_dims=10, rot_base=1e5, v_mix=True),
                     Moe(experts=13, top=2, ff=30, identity=2, group_count=5, group_keep=3, shared_ff=20)))),
        page=16, seed=54),
    # a larger one for long prompts: windows over several pages, key rows of exactly 128 entries and of more
    "e": dict(cfg=PemuvikConfig(vocab=384, width=192, eps=1e-5, layers=(
        PemuvikLayer("attention", Att(4, 2, 64, 48, 0.11, window=150, rot_dims=32, rot_base=2e4, v_mix=True),
                     Moe(experts=10, top=3, ff=72, identity=2, group_count=4, group_keep=2, shared_ff=48)),
        PemuvikLayer("latent_attention", Lat(heads=4, dim=48, rot_dim=32, vdim=48, kv_rank=96, scale=0.1, rot_base=2e4), 256),
        PemuvikLayer("attention", Att(6, 2, 32, 48, 0.15, window=70, rot_dims=32, rot_base=2e4, v_mix=True), 256),
        PemuvikLayer("latent_attention", Lat(heads=3, dim=64, rot_dim=16, vdim=32, kv_rank=176, scale=0.09, rot_base=1e5),
                     Moe(experts=10, top=3, ff=72, identity=2, group_count=4, group_keep=2, shared_ff=48)))),
        page=64, seed=55),
}

_folders: Dict[str, str] = {}
_tmp = None


def stretch(tensors: Dict[str, torch.Tensor], seed: int, sharp: bool = True) -> Dict[str, torch.Tensor]:
    """Random weights of N(0, std) hide faults: norms and layer scales at their neutral values, sinks and score
    biases at zero, a mixing factor of zero, router scores that all lie together, biases too small to be missed.
    This makes them of a size that shows.  sharp: also peaked scores and router logits far apart, which the float32
    tests want (a lost key or a wrong expert then moves the logits) and which multiply bfloat16's rounding."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for k, t in tensors.items():
        f = t.float()
        draw = lambda *shape: torch.randn(shape or f.shape, generator=gen)
        if k.endswith(".sink"):
            f = draw() * 1.5 + 0.5
        elif k.endswith(".pb"):
            f = draw() * 1.0 - 0.5
        elif k.endswith(".vmix"):
            f = 0.2 + 0.6 * torch.rand(f.shape, generator=gen)
        elif k.endswith(".router"):
            f = draw() * (0.6 if sharp else 0.15)
        elif k.endswith(".correction"):
            f = draw() * 0.08
        elif k.endswith(".sg"):
            f = draw() * 0.5
        elif k.endswith(".b"):
            f = draw() * 0.3
        elif k.endswith("norm1") or k.endswith("norm2") or k == "final.norm" or k.endswith(".norm") or k.endswith("ls1") \
                or k.endswith("ls2"):
            f = 1.0 + 0.4 * draw()
        elif sharp and (k.endswith(".mix.q") or k.endswith(".mix.k") or k.endswith(".mix.dkv")):
            f = f * 3.0
        out[k] = f.to(t.dtype).contiguous()
    return out


def model_folder(name: str, dtype: str = "float32") -> str:
    global _tmp
    key = f"{name}-{dtype}"
    if key not in _folders:
        if _tmp is None:
            _tmp = tempfile.TemporaryDirectory(prefix="nva-pemuvik-")
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


def paged_batch(dev, page, lens, q_lens, seed, window=None, free_passed=False, spare=2):
    """The step of requests that hold `lens` tokens after it, the last q_lens of which are its queries: block tables
    over shuffled pages (with free_passed the pages wholly before the window of a request's first query are taken out
    of its table, as the cache manager gives them back), the slot of every query's own key, and the slots of all
    earlier tokens (for filling a cache by hand).  Returns (batch, slots of this step's tokens, slots of every token
    per request or -1 where its page went back, number of pages)."""
    rng = random.Random(seed)
    S = len(lens)
    pages_per = [(n + page - 1) // page for n in lens]
    total = sum(pages_per) + spare
    order = list(range(total))
    rng.shuffle(order)
    tables = torch.full((S, max(pages_per)), -1, dtype=torch.int32)
    all_slots, step_slots, token_seq, positions = [], [], [], []
    for s, n in enumerate(lens):
        mine = [order.pop() for _ in range(pages_per[s])]
        held = set(range(len(mine)))
        if free_passed and window is not None:
            held = set(range(max(0, (n - q_lens[s]) - window + 1) // page, len(mine)))
        for p in held:
            tables[s, p] = mine[p]
        slots = [mine[j // page] * page + j % page if j // page in held else -1 for j in range(n)]
        all_slots.append(slots)
        step_slots += slots[n - q_lens[s]:]
        token_seq += [s] * q_lens[s]
        positions += list(range(n - q_lens[s], n))
    assert all(a == 1 or b != 1 for a, b in zip(q_lens, q_lens[1:])), "single tokens come first in a batch"
    batch = SimpleNamespace(
        num_seqs=S, num_tokens=sum(q_lens), token_seq=torch.tensor(token_seq, dtype=torch.int32, device=dev),
        positions=torch.tensor(positions, dtype=torch.int32, device=dev), max_kv_len=max(lens), max_q_len=max(q_lens),
        kv_lens=torch.tensor(lens, dtype=torch.int32, device=dev),
        cu_seqlens_q=torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32, device=dev),
        num_decode=next((i for i, n in enumerate(q_lens) if n != 1), len(q_lens)), q_lens=list(q_lens),
        starts=[n - m for n, m in zip(lens, q_lens)], step_cache={},
        groups=[SimpleNamespace(block_tables=tables.to(dev),
                                slot_mapping=torch.tensor(step_slots, dtype=torch.int32, device=dev))])
    return batch, step_slots, all_slots, total


def fill_cache(kc, vc, slots, keys, values):
    """keys [n, G, D], values [n, G, DV] of one request into the slots of its tokens (-1: the page went back)."""
    page, vt = kc.shape[2], vc.shape[4]
    for j, s in enumerate(slots):
        if s >= 0:
            kc[s // page, :, s % page, :] = keys[j].to(kc.device)
            vc[s // page, :, (s % page) // vt, :, (s % page) % vt] = values[j].to(vc.device)
