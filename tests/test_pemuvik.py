"""Pemuvik: every mechanism alone, and the model through the step function and the engine, against
the plain implementation (tests/plain_pemuvik.py).  Each test runs on the CPU stand-ins of the
device operations (tests/torch_kernels.py; this checks the stand-ins and the host logic) and, marked
gpu, on the HIP kernels."""
import json
import math

import pytest
import torch

import helpers as H
import pemuvik_cases as K
import plain_pemuvik as plain
from nano_vllm_amd import LLM, SamplingParams
from nano_vllm_amd.config import ConfigError, PemuvikConfig, architecture_of
from torch_kernels import TorchKernels, new_caches

BACKENDS = ["cpu", pytest.param("hip", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
_hip = {}


def _kernels(backend, dtype=torch.float32):
    if backend == "cpu":
        return TorchKernels("cpu", dtype), "cpu"
    from nano_vllm_amd.kernels import HipKernels
    if dtype not in _hip:
        _hip[dtype] = HipKernels("cuda:0", dtype, quiet=True)
    return _hip[dtype], "cuda:0"


def _tol(dtype):
    return 3e-5 if dtype == torch.float32 else 2e-2


def _close(got, want, dtype, what="", tol=None):
    e = float((got.double().cpu() - want.double()).abs().max() / max(float(want.double().abs().max()), 1e-9))
    assert e < (tol or _tol(dtype)), f"{what}: differs by {e:.2e} of the largest"


# ------------------------------------------------------------------------------ configuration
def test_config_is_read_written_and_refused():
    for name, c in K.CONFIGS.items():
        d = c["cfg"].to_dict()
        arch = architecture_of(d)
        assert arch.name == "Pemuvik"
        again = arch.parse_config(json.loads(json.dumps(d)))
        assert again == c["cfg"].__class__(**{**c["cfg"].__dict__, "dtype": again.dtype}), name
    d = K.CONFIGS["a"]["cfg"].to_dict()
    # what may be left out: the mask, the rotation, the mixing of values, identities, groups, the shared expert
    e = json.loads(json.dumps(d))
    e["layers"][0]["mixer"].pop("mask"), e["layers"][0]["mixer"].pop("rot"), e["layers"][0]["mixer"].pop("v_mix")
    router = e["layers"][1]["mlp"]["router"]
    router.pop("identity"), router.pop("groups")
    e["layers"][1]["mlp"].pop("shared")
    got = PemuvikConfig.from_dict(e)
    m, f = got.layers[0].mixer, got.layers[1].mlp
    assert (m.window, m.rot_dims, m.v_mix) == (None, 0, False)
    assert (f.identity, f.group_count, f.group_keep, f.shared_ff) == (0, 1, 1, None)
    assert got.layers[4].mlp is None and got.layers[0].mlp == 40

    def broken(change):
        x = json.loads(json.dumps(d))
        change(x)
        with pytest.raises(ConfigError):
            PemuvikConfig.from_dict(x)
    broken(lambda x: x["layers"][0].update(type="retention"))
    broken(lambda x: x["layers"][0]["mixer"].update(heads=3))                   # 3 heads on 2 kv heads
    broken(lambda x: x["layers"][0]["mixer"]["rot"].update(dims=7))
    broken(lambda x: x["layers"][0]["mixer"]["rot"].update(dims=18))            # more than the head
    broken(lambda x: x["layers"][1]["mixer"].update(vdim=8))                    # mixed values of another size
    broken(lambda x: x["layers"][2]["mixer"]["rot"].update(dims=4))             # not the latent layer's rot_dim
    broken(lambda x: x["layers"][2]["mixer"].pop("kv_rank"))
    broken(lambda x: x["layers"][1]["mlp"]["router"].update(top=5))             # 2 groups of 2 hold 4
    broken(lambda x: x["layers"][1]["mlp"]["router"]["groups"].update(count=3))  # 8 outputs in 3 groups
    broken(lambda x: x["layers"][1]["mlp"].update(kind="sparse"))
    broken(lambda x: x["norm"].update(eps=0.0))
    broken(lambda x: x.pop("vocab"))


def test_the_checkpoint_is_read_by_its_own_names():
    from safetensors import safe_open
    with safe_open(K.model_folder("a") + "/model.safetensors", "pt", "cpu") as f:
        names = set(f.keys())
        shapes = {n: tuple(f.get_slice(n).get_shape()) for n in names}
    for n in ("embed", "final.norm", "l0.norm1", "l0.norm2", "l0.ls1", "l0.ls2", "l0.mix.q", "l0.mix.q.b", "l0.mix.k.b",
              "l0.mix.v.b", "l0.mix.o.b", "l0.mix.vmix", "l0.mix.pb", "l0.mlp.gate", "l0.mlp.up", "l0.mlp.down", "l1.mlp.router",
              "l1.mlp.correction", "l1.mlp.e5.gate", "l1.mlp.e0.down", "l1.mlp.shared.gate", "l1.mlp.shared.sg", "l2.mix.q",
              "l2.mix.dkv", "l2.mix.dkv.norm", "l2.mix.uk", "l2.mix.uv", "l2.mix.sink", "l2.mix.o", "l4.ls1", "l5.norm1"):
        assert n in names, n
    assert not {"head", "l4.norm2", "l4.ls2", "l3.mix.vmix", "l1.mlp.e6.gate", "l2.mix.o.b"} & names
    assert shapes["l0.mix.vmix"] == () and shapes["l1.mlp.router"] == (8, 48) and shapes["l1.mlp.correction"] == (8,)
    assert shapes["l1.mlp.shared.sg"] == (1, 48) and shapes["l2.mix.dkv"] == (26, 48) and shapes["l2.mix.uk"] == (30, 20)
    assert shapes["l2.mix.uv"] == (42, 20) and shapes["l2.mix.q"] == (48, 48)


# ------------------------------------------------------------------------------ the block's norms
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [48, 20, 328, 1000])
def test_two_norms_of_one_stream_and_scaled_addends(backend, dtype, width):
    k, dev = _kernels(backend, dtype)
    g = torch.Generator().manual_seed(width)
    rows = 5
    stream = (torch.randn((rows, width), generator=g) * 300.0).to(dev)          # far beyond bfloat16's grain
    a, b = (torch.randn((rows, width), generator=g).to(dtype).to(dev) for _ in range(2))
    sa, sb, w1, w2 = ((1.0 + 0.5 * torch.randn(width, generator=g)).to(dtype).to(dev) for _ in range(4))
    want_stream = stream.double().cpu() + a.double().cpu() * sa.double().cpu() + b.double().cpu() * sb.double().cpu()
    unit = plain.unit_mean(want_stream, 1e-5)
    res = stream.clone()
    y1, y2, res = k.stream_scaled_norm([(a, sa), (b, sb)], res, w1, 1e-5, weight2=w2)
    _close(res, want_stream, torch.float32, "stream")
    _close(y1, unit * w1.double().cpu(), dtype, "first norm")
    _close(y2, unit * w2.double().cpu(), dtype, "second norm")
    # one addend and one norm; no addend at all; a stream that starts with an unscaled addend
    res2 = stream.clone()
    y, none, res2 = k.stream_scaled_norm([(a, sa)], res2, w1, 1e-5)
    assert none is None
    _close(res2, stream.double().cpu() + a.double().cpu() * sa.double().cpu(), torch.float32, "one addend")
    y, y2, same = k.stream_scaled_norm([], res2, w1, 1e-5, weight2=w2, dtype=dtype)
    _close(y2, plain.unit_mean(res2.double().cpu(), 1e-5) * w2.double().cpu(), dtype, "no addend")
    y, _, started = k.stream_scaled_norm([(a, None)], None, w2, 1e-5)
    assert started.dtype == torch.float32
    _close(started, a.double().cpu(), torch.float32, "start")
    _close(y, plain.unit_mean(a.double().cpu(), 1e-5) * w2.double().cpu(), dtype, "start's norm")


# ------------------------------------------------------------------------------ preparation of q, k, v
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,D,DV,R,page", [(4, 2, 16, 24, 8, 8), (2, 2, 24, 8, 24, 4), (3, 1, 10, 10, 0, 16), (8, 2, 64, 64, 32, 32),
                                                (1, 1, 6, 10, 2, 4)])
def test_neighbouring_pairs_turn_values_are_normed_and_mixed_then_stored(backend, dtype, hq, hkv, D, DV, R, page):
    k, dev = _kernels(backend, dtype)
    g = torch.Generator().manual_seed(hq * 100 + D)
    positions = [0, 1, 2, 7, 63, 64, 1000, 29999, 30000]
    T = len(positions)
    eps = 1e-5
    width = (hq + hkv) * D + hkv * DV
    qkv = (torch.randn((T, width), generator=g) * 2.0).to(dtype)
    lam = torch.tensor(0.3, dtype=torch.float32)
    base = 1e4
    inv_freq = 1.0 / (base ** (torch.arange(0, R, 2, dtype=torch.float) / R)) if R else None
    pos = torch.tensor(positions, dtype=torch.int32, device=dev)
    table = k.rotary_step_table(inv_freq.to(dev), pos) if R else None
    slots = torch.tensor([3, 0, 9, 17, 5, -1, 11, 2, 20], dtype=torch.int32, device=dev)
    x = qkv.double()
    q, kk = x[:, :hq * D].view(T, hq, D), x[:, hq * D:(hq + hkv) * D].view(T, hkv, D)
    v = plain.unit_mean(x[:, (hq + hkv) * D:].view(T, hkv, DV), eps)

    def turned(y):
        if not R:
            return y
        return torch.stack([plain.turn_pairs(y[t:t + 1], {"dims": R, "base": base}, positions[t])[0] for t in range(T)])
    for first in (True, False):
        kc, vc = new_caches(24 // page + 1 if page <= 8 else 2, hkv, D, page, dtype, dev, v_head_dim=DV)
        kc.fill_(float("nan")), vc.fill_(float("nan"))
        row = qkv.clone().to(dev)
        v_first = torch.randn((T, hkv * DV), generator=g).to(dev)
        extra = dict(v_first_out=torch.full((T, hkv * DV), float("nan"), device=dev)) if first else dict(v_first_in=v_first, v_mix=lam.to(dev))
        ok = slots.cpu() >= 0
        s = slots.cpu()[ok].long() % (kc.shape[0] * page)
        use = slots.clone()
        use[ok.to(dev)] = s.to(torch.int32).to(dev)
        got_q = k.qk_rownorm_store(row, hq, hkv, D, DV, None, None, eps, pos, 0.0, 1, use, kc, vc, rot_table=table,
                                   rot_interleaved=True, v_norm=True, **extra)
        # (angles are float32 products p * f: their rounding grows with the position)
        for t in range(T):
            _close(got_q.reshape(T, hq, D)[t], turned(q)[t], dtype, f"q of token {t}", tol=_tol(dtype) + 2.5e-7 * positions[t])
        want_v = v if first else (1.0 - 0.3) * v + 0.3 * v_first.double().cpu().view(T, hkv, DV)
        if first:
            _close(extra["v_first_out"].view(T, hkv, DV), v, torch.float32, "the first layer's values", tol=3e-5 if dtype == torch.float32 else 1e-6 + 1e-2)
        vt = vc.shape[4]
        for t in range(T):
            if not bool(ok[t]):
                continue
            sl = int(use[t])
            _close(kc[sl // page, :, sl % page, :], turned(kk)[t], dtype, f"k of token {t}", tol=_tol(dtype) + 2.5e-7 * positions[t])
            _close(vc[sl // page, :, (sl % page) // vt, :, (sl % page) % vt], want_v[t], dtype, f"v of token {t}")


# ------------------------------------------------------------------------------ window attention with sigmoid weights
def _sigmoid_case(dtype, dev, hq, hkv, D, DV, page, lens, q_lens, seed, window, boost=None, free_passed=False):
    g = torch.Generator().manual_seed(seed)
    batch, _, all_slots, pages = K.paged_batch(dev, page, lens, q_lens, seed, window, free_passed)
    kc, vc = new_caches(pages, hkv, D, page, dtype, dev, v_head_dim=DV)
    kc.fill_(float("nan")), vc.fill_(float("nan"))
    qs, ks, vs = [], [], []
    for s, n in enumerate(lens):
        kk = torch.randn((n, hkv, D), generator=g).to(dtype)
        vv = torch.randn((n, hkv, DV), generator=g).to(dtype)
        qq = torch.randn((n, hq, D), generator=g).to(dtype)
        if boost is not None and boost[0] == s:
            # one key that its request's queries prefer by far, all others far below the sigmoid's middle
            kk[:] = 0
            kk[:, :, 1] = -8.0
            kk[boost[1]] = 0
            kk[boost[1], :, 0] = 8.0
            qq[:] = 0
            qq[:, :, 0] = 8.0
            qq[:, :, 1] = 8.0
        K.fill_cache(kc, vc, all_slots[s], kk, vv)
        qs.append(qq), ks.append(kk), vs.append(vv)
    q = torch.cat([qs[s][lens[s] - q_lens[s]:] for s in range(len(lens))]).reshape(sum(q_lens), hq * D).contiguous().to(dev)
    return q, kc, vc, batch, (qs, ks, vs)


def _plain_sigmoid(qs, ks, vs, lens, q_lens, scale, window, bias):
    m = {"scale": scale, "mask": None if window is None else {"size": window}}
    rows = []
    for q, k, v, n, c in zip(qs, ks, vs, lens, q_lens):
        o = plain.sigmoid_window_attend(q.double(), k.double(), v.double(), m, bias.double(), rows=range(n - c, n))
        rows.append(o[n - c:])
    return torch.cat(rows)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,D,DV,page,window,lens,q_lens", [
    (4, 2, 16, 24, 8, 10, [30, 9, 41], [1, 1, 41]),            # single tokens beside a whole prompt
    (2, 2, 24, 8, 4, 21, [50, 33], [17, 33]),                 # a portion behind 33 cached tokens
    (3, 1, 8, 8, 16, 1, [20, 5], [1, 5]),                     # a window of one position: the token itself
    (6, 2, 64, 64, 32, 48, [130, 70, 100], [1, 2, 64]),       # equal head sizes: the matrix cores' kernels in bfloat16
    (8, 2, 128, 128, 64, 100, [300, 1, 150, 400], [1, 1, 1, 130]),
    (2, 1, 10, 10, 4, None, [37, 12], [1, 12]),               # no window
    (4, 2, 16, 24, 8, 200, [90], [30]),                       # a window longer than the request
    (2, 1, 32, 48, 64, 70, [300, 260], [1, 100]),             # windows over page borders
])
def test_window_attention_with_sigmoid_weights(backend, dtype, hq, hkv, D, DV, page, window, lens, q_lens):
    k, dev = _kernels(backend, dtype)
    bias = torch.tensor([0.5, -1.0, 0.0, 2.0, -0.3, 1.1, -2.0, 0.7][:hq], dtype=torch.float32)
    scale = 0.3
    for free_passed in (False, True):
        q, kc, vc, batch, (qs, ks, vs) = _sigmoid_case(dtype, dev, hq, hkv, D, DV, page, lens, q_lens, 7, window, free_passed=free_passed)
        got = k.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, scale, window, v_head_dim=DV, sigmoid_bias=bias.to(dev))
        k.check_faults()
        want = _plain_sigmoid(qs, ks, vs, lens, q_lens, scale, window, bias)
        _close(got, want, dtype, f"free_passed={free_passed}")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,DV,page", [(16, 24, 8), (64, 64, 64)])
def test_a_key_just_inside_and_just_outside_the_window(backend, dtype, D, DV, page):
    """One key carries nearly all the weight its request gives.  A query whose window still holds it returns that
    key's value; the next query returns nearly nothing (the weights are not normalised: nothing takes its place)."""
    k, dev = _kernels(backend, dtype)
    hq, hkv, window = 2, 1, 23
    bias = torch.zeros(hq, dtype=torch.float32)
    for n, portion in ((200, 1), (200, 60), (90, 90)):
        for back in (window - 1, window):                      # the favourite key lies `back` positions before the last query
            fav = n - 1 - back
            q, kc, vc, batch, (qs, ks, vs) = _sigmoid_case(dtype, dev, hq, hkv, D, DV, page, [n], [portion], 11, window,
                                                           boost=(0, fav), free_passed=True)
            got = k.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, 1.0, window, v_head_dim=DV, sigmoid_bias=bias.to(dev))
            k.check_faults()
            last = got[-1].float().cpu().view(hq, DV)
            value = vs[0][fav, 0].float()
            if back < window:
                assert float((last - value).abs().max()) < 0.05 * float(value.abs().max()) + 1e-3, (n, portion, back)
            else:
                assert float(last.abs().max()) < 1e-3, (n, portion, back)
            want = _plain_sigmoid(qs, ks, vs, [n], [portion], 1.0, window, bias)
            _close(got, want, dtype, f"{(n, portion, back)}", tol=None if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_score_bias_and_the_missing_normalisation_show(backend):
    """Keys of score zero: every one weighs sigmoid(bias), so the output is the number of visible keys times that,
    times the values' mean: it grows with the window where a softmax's would not."""
    k, dev = _kernels(backend, torch.float32)
    hq, hkv, D, DV, page, n, window = 2, 1, 8, 4, 8, 40, 16
    batch, _, all_slots, pages = K.paged_batch(dev, page, [n], [n], 3, window)
    kc, vc = new_caches(pages, hkv, D, page, torch.float32, dev, v_head_dim=DV)
    K.fill_cache(kc, vc, all_slots[0], torch.zeros(n, hkv, D), torch.ones(n, hkv, DV))
    q = torch.randn(n, hq * D).to(dev)
    bias = torch.tensor([-2.0, 1.0])
    got = k.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, 0.5, window, v_head_dim=DV, sigmoid_bias=bias.to(dev)).cpu()
    for i in (0, 5, 15, 16, 39):
        seen = min(i + 1, window)
        for h in range(hq):
            assert abs(float(got[i, h * DV]) - seen / (1.0 + math.exp(-float(bias[h])))) < 1e-4, (i, h)


# ------------------------------------------------------------------------------ attention through a latent
def _latent_case(dtype, dev, H_, D, R, DV, C, page, lens, q_lens, seed, boost=None):
    g = torch.Generator().manual_seed(seed)
    batch, step_slots, all_slots, pages = K.paged_batch(dev, page, lens, q_lens, seed)
    kc, vc = new_caches(pages, 1, C + R, page, dtype, dev, v_head_dim=C)
    kc.fill_(float("nan")), vc.fill_(float("nan"))
    width = H_ * (D + R) + C + R
    rows = [(torch.randn((n, width), generator=g) * 1.5).to(dtype) for n in lens]
    w = {"uk": (torch.randn((H_ * D, C), generator=g) * 0.4).to(dtype), "uv": (torch.randn((H_ * DV, C), generator=g) * 0.4).to(dtype),
         "norm": (1.0 + 0.3 * torch.randn(C, generator=g)).to(dtype), "sink": torch.randn(H_, generator=g) * 2.0}
    if boost is not None:
        # (the latent is normed: a row stands out by its direction, not its size.)  Every latent points along
        # channel 0 but one, which points along channel 1; the keys' plain parts copy the latent's first channels and
        # every query asks for channel 1 alone: that row scores about 10, all others 0.
        s, j = boost
        lat = H_ * (D + R)
        rows[s][:] = 0
        rows[s][:, lat] = 1.0
        rows[s][j, lat], rows[s][j, lat + 1] = 0.0, 1.0
        for h in range(H_):
            rows[s][:, h * (D + R) + 1] = 6.0
        w["uk"][:] = 0
        for h in range(H_):
            for i in range(min(D, C)):
                w["uk"][h * D + i, i] = 1.0
        w["norm"][:] = 1.0
    return batch, all_slots, kc, vc, rows, w


def _plain_latent(rows, w, H_, D, R, DV, C, scale, eps, base, lens, q_lens):
    out = []
    for x, n, c in zip(rows, lens, q_lens):
        x = x.double()
        q = x[:, :H_ * (D + R)].view(n, H_, D + R)
        qp, qt = q[:, :, :D], plain.turn_pairs(q[:, :, D:], {"dims": R, "base": base})
        lat = plain.unit_mean(x[:, H_ * (D + R):H_ * (D + R) + C], eps) * w["norm"].double()
        kt = plain.turn_pairs(x[:, H_ * (D + R) + C:].reshape(n, 1, R), {"dims": R, "base": base})[:, 0]
        kp = (lat @ w["uk"].double().T).view(n, H_, D)
        v = (lat @ w["uv"].double().T).view(n, H_, DV)
        o = torch.zeros(n, H_, DV, dtype=torch.float64)
        for h in range(H_):
            for i in range(n - c, n):
                s = (kp[:i + 1, h] @ qp[i, h] + kt[:i + 1] @ qt[i, h]) * scale
                o[i, h] = plain.sink_softmax_rows(s, w["sink"][h]) @ v[:i + 1, h]
        out.append(o[n - c:].reshape(c, -1))
    return torch.cat(out)


def _run_latent(k, dev, dtype, batch, all_slots, kc, vc, rows, w, H_, D, R, DV, C, scale, eps, base, lens, q_lens):
    """The cache is filled by earlier steps of the same operations, then the step at hand runs."""
    inv_freq = (1.0 / (base ** (torch.arange(0, R, 2, dtype=torch.float) / R))).to(dev)
    for s, n in enumerate(lens):                                         # the tokens before this step, request by request
        before = n - q_lens[s]
        if before:
            pos = torch.arange(before, dtype=torch.int32, device=dev)
            k.latent_prepare(rows[s][:before].to(dev), H_, D, R, C, w["norm"].to(dev), eps, k.rotary_step_table(inv_freq, pos),
                             torch.tensor(all_slots[s][:before], dtype=torch.int32, device=dev), kc, vc)
    proj = torch.cat([rows[s][lens[s] - q_lens[s]:] for s in range(len(lens))]).to(dev)
    q2 = k.latent_prepare(proj, H_, D, R, C, w["norm"].to(dev), eps, k.rotary_step_table(inv_freq, batch.positions),
                          batch.groups[0].slot_mapping, kc, vc)
    k.heads_linear(proj, D + R, w["uk"].to(dev), H_, C, D, True, q2, C + R)
    o = k.latent_attention(q2, H_, C, R, kc, vc, batch, 0, scale, sinks=w["sink"].to(dev))
    k.check_faults()
    heads = o.new_empty((o.shape[0], H_ * DV))
    k.heads_linear(o, C, w["uv"].to(dev), H_, DV, C, False, heads, DV)
    return heads


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H_,D,R,DV,C,page,lens,q_lens", [
    (3, 10, 6, 14, 20, 8, [30, 9, 41], [1, 1, 41]),
    (1, 4, 2, 6, 5, 4, [13, 6], [1, 6]),
    (4, 32, 32, 32, 64, 32, [130, 70], [2, 70]),
    (2, 24, 16, 40, 16, 16, [50, 33], [17, 33]),
    (2, 64, 16, 32, 176, 64, [100], [37]),                    # key rows of more than 128 entries
    (2, 16, 32, 16, 96, 64, [1, 200], [1, 150]),              # key rows of exactly 128, the first token of a sequence
    (20, 32, 64, 32, 384, 64, [1500, 33, 700], [1, 1, 40]),   # more heads than a tile of columns, shares of a token's keys
    (5, 24, 24, 40, 80, 32, [1000, 2], [1, 1]),               # a key row that ends inside a step of 32 channels
])
def test_attention_through_a_latent(backend, dtype, H_, D, R, DV, C, page, lens, q_lens):
    k, dev = _kernels(backend, dtype)
    scale, eps, base = 0.2, 1e-5, 1e3
    batch, all_slots, kc, vc, rows, w = _latent_case(dtype, dev, H_, D, R, DV, C, page, lens, q_lens, 5)
    got = _run_latent(k, dev, dtype, batch, all_slots, kc, vc, rows, w, H_, D, R, DV, C, scale, eps, base, lens, q_lens)
    want = _plain_latent(rows, w, H_, D, R, DV, C, scale, eps, base, lens, q_lens)
    # (angles are float32 products p * f: their rounding grows with the position)
    _close(got, want, dtype, "latent attention", tol=1e-4 if dtype == torch.float32 else 4e-2)


@pytest.mark.parametrize("backend", BACKENDS)
def test_a_far_key_among_hundreds_and_the_sink(backend):
    """One latent row 700 positions back stands out among flat ones: the last query's output follows it, for a whole
    prompt, a portion and a single token; a sink far above every score takes the weight away, one far below changes
    nothing."""
    k, dev = _kernels(backend, torch.float32)
    H_, D, R, DV, C, page = 2, 8, 4, 6, 12, 16
    n, fav = 760, 60
    outs = {}
    for sink in (-60.0, 0.0, 40.0):
        for portion in (n, 64, 1):
            batch, all_slots, kc, vc, rows, w = _latent_case(torch.float32, dev, H_, D, R, DV, C, page, [n], [portion], 9, boost=(0, fav))
            w["sink"] = torch.full((H_,), sink)
            got = _run_latent(k, dev, torch.float32, batch, all_slots, kc, vc, rows, w, H_, D, R, DV, C, 0.5, 1e-5, 1e3, [n], [portion])
            want = _plain_latent(rows, w, H_, D, R, DV, C, 0.5, 1e-5, 1e3, [n], [portion])
            _close(got, want, torch.float32, f"sink {sink}, portion {portion}")
            outs[(sink, portion)] = got[-1].cpu()
    assert float((outs[(-60.0, 1)] - outs[(0.0, 1)]).abs().max()) < 1e-3 * float(outs[(-60.0, 1)].abs().max())
    assert float(outs[(40.0, 1)].abs().max()) < 1e-3 * float(outs[(-60.0, 1)].abs().max())
    # without the far key the output differs: it was seen
    batch, all_slots, kc, vc, rows, w = _latent_case(torch.float32, dev, H_, D, R, DV, C, page, [n], [1], 9, boost=(0, fav))
    w["sink"] = torch.full((H_,), -60.0)
    lat = H_ * (D + R)
    rows[0][fav, lat:lat + C] = rows[0][fav + 1, lat:lat + C]
    flat = _run_latent(k, dev, torch.float32, batch, all_slots, kc, vc, rows, w, H_, D, R, DV, C, 0.5, 1e-5, 1e3, [n], [1])
    assert float((flat[-1].cpu() - outs[(-60.0, 1)]).abs().max()) > 0.05 * float(outs[(-60.0, 1)].abs().max())


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,heads,n_out,k_in,transposed", [(1, 3, 20, 10, True), (37, 2, 7, 13, False), (16, 4, 64, 32, True),
                                                                (70, 1, 130, 176, False), (5, 6, 96, 48, True)])
def test_a_product_per_head(backend, dtype, tokens, heads, n_out, k_in, transposed):
    k, dev = _kernels(backend, dtype)
    g = torch.Generator().manual_seed(tokens + n_out)
    x_head, y_head, off = k_in + 5, n_out + 3, 2
    x = torch.randn((tokens, heads * x_head), generator=g).to(dtype)
    w = torch.randn((heads * k_in, n_out) if transposed else (heads * n_out, k_in), generator=g).to(dtype)
    y = torch.zeros((tokens, heads * y_head + off), dtype=dtype, device=dev)
    k.heads_linear(x.to(dev), x_head, w.to(dev), heads, n_out, k_in, transposed, y, y_head, off)
    for h in range(heads):
        wh = w[h * k_in:(h + 1) * k_in].double().T if transposed else w[h * n_out:(h + 1) * n_out].double()
        want = x[:, h * x_head:h * x_head + k_in].double() @ wh.T
        _close(y[:, off + h * y_head: off + h * y_head + n_out], want, dtype, f"head {h}")
        assert float(y[:, off + h * y_head + n_out: off + (h + 1) * y_head].abs().max()) == 0.0 if h + 1 < heads else True


# ------------------------------------------------------------------------------ the routed feed-forward
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,identity,top,count,keep", [(6, 2, 3, 4, 2), (5, 0, 2, 1, 1), (1, 0, 1, 1, 1), (2, 1, 3, 1, 1), (13, 2, 2, 5, 3),
                                                             (8, 4, 3, 3, 2), (60, 4, 6, 8, 3), (3, 0, 3, 3, 3)])
def test_the_choice_by_corrected_scores_within_the_best_groups(backend, experts, identity, top, count, keep):
    k, dev = _kernels(backend)
    g = torch.Generator().manual_seed(experts * 10 + top)
    n, T = experts + identity, 40
    z = torch.randn((T, n + 3), generator=g) * 2.0                     # (wider rows: the logits are their first columns)
    # negative choice scores throughout: an expert outside the kept groups must not count as zero
    correction = torch.randn(n, generator=g) * 0.05 - (0.6 if experts % 2 else 0.0)
    router = {"experts": experts, "identity": identity, "top": top, "groups": {"count": count, "keep": keep}}
    ids, weights = k.moe_route(z.to(dev)[:, :n], top, count, keep, 1.0, routing="softmax_choice", bias=correction.to(dev))
    for t in range(T):
        s = torch.softmax(z[t, :n].double(), dim=-1)
        picked, w = plain.chosen_experts(s, correction.double(), router)
        assert ids[t].tolist() == picked, (t, ids[t].tolist(), picked)
        assert float((weights[t].double().cpu() - w).abs().max()) < 1e-6
        assert abs(float(weights[t].sum()) - 1.0) < 1e-5


@pytest.mark.parametrize("backend", BACKENDS)
def test_a_token_whose_best_expert_sits_in_a_poor_group(backend):
    k, dev = _kernels(backend)
    # groups {0,1}, {2,3}, {4,5}: expert 2 has the third best score, but the two best groups are the first and the last
    z = torch.log(torch.tensor([[0.30, 0.02, 0.20, 0.01, 0.25, 0.22]]))
    ids, weights = k.moe_route(z.to(dev), 3, 3, 2, 1.0, routing="softmax_choice", bias=torch.zeros(6).to(dev))
    assert ids[0].tolist() == [0, 4, 5]
    assert float((weights[0].cpu() - torch.tensor([0.30, 0.25, 0.22]) / 0.77).abs().max()) < 1e-6
    # the correction moves the choice and leaves the weights alone
    ids, weights = k.moe_route(z.to(dev), 2, 1, 1, 1.0, routing="softmax_choice", bias=torch.tensor([0., 0.5, 0., 0., 0., 0.]).to(dev))
    assert ids[0].tolist() == [1, 0]
    assert float((weights[0].cpu() - torch.tensor([0.02, 0.30]) / 0.32).abs().max()) < 1e-6


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,width,ff,experts,identity,top", [(1, 48, 20, 6, 2, 3), (7, 20, 9, 5, 0, 3), (150, 72, 30, 10, 2, 2),
                                                                  (33, 128, 64, 8, 4, 3), (300, 64, 32, 2, 1, 3)])
def test_gated_experts_identities_and_the_gated_shared_expert(backend, dtype, tokens, width, ff, experts, identity, top):
    k, dev = _kernels(backend, dtype)
    g = torch.Generator().manual_seed(tokens + width)
    x = torch.randn((tokens, width), generator=g).to(dtype)
    up = (torch.randn((experts * 2 * ff, width), generator=g) * 0.3).to(dtype)
    down = (torch.randn((experts * width, ff), generator=g) * 0.3).to(dtype)
    n = experts + identity
    ids = torch.stack([torch.randperm(n, generator=g)[:top] for _ in range(tokens)]).to(torch.int32)
    if identity and tokens > 2:
        ids[0, :min(top, identity)] = torch.arange(experts, experts + min(top, identity), dtype=torch.int32)   # identities only, if they suffice
    weights = torch.rand((tokens, top), generator=g)
    add = torch.randn((tokens, width), generator=g).to(dtype)
    gate = torch.randn((tokens, 3), generator=g) * 2.0
    got = k.moe_experts(x.to(dev), ids.to(dev), weights.to(dev), up.to(dev), down.to(dev), experts, "silu", add=add.to(dev), gated=True,
                        add_gate=gate.to(dev)[:, 1])
    w = {}
    for e in range(experts):
        w[f"e{e}.gate"], w[f"e{e}.up"] = up[2 * e * ff:(2 * e + 1) * ff].double(), up[(2 * e + 1) * ff:(2 * e + 2) * ff].double()
        w[f"e{e}.down"] = down[e * width:(e + 1) * width].double()
    want = torch.zeros((tokens, width), dtype=torch.float64)
    for t in range(tokens):
        for c in range(top):
            e = int(ids[t, c])
            want[t] += float(weights[t, c]) * (x[t].double() if e >= experts else plain.gated_unit(x[t].double(), w, f"e{e}.", plain.silu))
        want[t] += torch.sigmoid(gate[t, 1].double()) * add[t].double()
    _close(got, want, dtype, "experts", tol=None if dtype == torch.float32 else 3e-2)


# ------------------------------------------------------------------------------ the model through the step function
def _runner(name, backend, dtype, pages, max_requests=4):
    kernels, dev = _kernels(backend, torch.float32 if dtype == "float32" else torch.bfloat16)
    return H.make_runner(K.model_folder(name, dtype), dtype, K.CONFIGS[name]["page"], pages, device=dev,
                         kernels=kernels, max_requests=max_requests)


MODEL_TOL = {"float32": 1e-4, "bfloat16": 6e-2}


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_every_cutting_gives_the_plain_logits(backend, name):
    c = K.CONFIGS[name]
    n = 70 if (backend, name) == ("cpu", "b") else 110
    toks = H.random_tokens(c["cfg"].vocab, n, 1)
    want = K.plain_logits(K.model_folder(name), toks)
    r = _runner(name, backend, "float32", 40)
    windows = {l.mixer.window if l.kind == "attention" else None for l in c["cfg"].layers}
    assert len(r.cache.groups) == len(windows)
    for portions in (H.whole(n), H.last_one_by_one(n, 45), H.changing_portions(n, 2), [1] * 3 + [2] * 10 + [n - 23]):
        got = H.run_portions(r, "x", toks, portions)
        assert K.err(got, want) < MODEL_TOL["float32"], portions
    assert all(pool.num_free == 40 for pool in r.cache.pools)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["a", "b", "d"])
def test_bfloat16_follows_the_plain_logits_under_every_cutting(name):
    c = K.CONFIGS[name]
    n = 130
    toks = H.random_tokens(c["cfg"].vocab, n, 3)
    want = K.plain_logits(K.model_folder(name, "bfloat16"), toks)
    r = _runner(name, "hip", "bfloat16", 40)
    for portions in (H.whole(n), H.last_one_by_one(n, 40), H.changing_portions(n, 4)):
        e = K.errors(H.run_portions(r, "x", toks, portions), want)
        # bfloat16's rounding through the layers stays at a few hundredths of the logits' spread; where two choice
        # scores lie close it may give a token another expert: few positions
        assert float(e.median()) < 0.05 and float(e.quantile(0.95)) < 0.35 and float(e.max()) < 1.0, \
            (portions, float(e.median()), float(e.quantile(0.95)), float(e.max()))


@pytest.mark.gpu
def test_a_larger_model_over_long_prompts():
    """Six hundred tokens through a model with windows over several pages and key rows of 128 entries and more:
    whole, in changing portions, and its last tokens one by one."""
    name = "e"
    c = K.CONFIGS[name]
    n = 600
    toks = H.random_tokens(c["cfg"].vocab, n, 17)
    want = K.plain_logits(K.model_folder(name), toks)
    r = _runner(name, "hip", "float32", 12)
    assert len(r.cache.groups) == 3
    for portions in (H.whole(n), H.changing_portions(n, 5), H.last_one_by_one(n, 180)):
        assert K.err(H.run_portions(r, "x", toks, portions), want) < MODEL_TOL["float32"], portions[:4]
    assert all(pool.num_free == 12 for pool in r.cache.pools)


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_first_tokens_of_a_sequence(backend):
    for name in ("a", "c"):
        c = K.CONFIGS[name]
        r = _runner(name, backend, "float32", 8)
        for n in (1, 2, 3, 5):
            toks = H.random_tokens(c["cfg"].vocab, n, 40 + n)
            want = K.plain_logits(K.model_folder(name), toks)
            for portions in ([n], [1] * n):
                assert K.err(H.run_portions(r, "x", toks, portions), want) < MODEL_TOL["float32"], (name, n, portions)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["a", "c"])
def test_long_decoding(backend, name):
    # one prompt token, then 170 tokens one by one: every window passes over decoded tokens, the latent layers see them all
    c = K.CONFIGS[name]
    n = 171
    toks = H.random_tokens(c["cfg"].vocab, n, 5)
    want = K.plain_logits(K.model_folder(name), toks)
    r = _runner(name, backend, "float32", 48)
    assert K.err(H.run_portions(r, "x", toks, [1] * n), want) < MODEL_TOL["float32"]
    if name == "a":
        # a window's group holds the pages of its window only, the latent layers' group all of them
        r.cache.admit("y")
        for pos in range(n):
            r.cache.reserve("y", pos + 1)
        by_window = {g.window: sum(1 for p in t if p >= 0) for g, t in zip(r.cache.groups, r.cache.requests["y"].tables)}
        assert by_window[10] <= 3 and by_window[21] <= 4 and by_window[7] <= 2 and by_window[33] <= 6 and by_window[None] == 22, by_window
        r.cache.release("y")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["a", "d"])
def test_mixed_batches_on_pages_that_are_used_again(backend, name):
    c = K.CONFIGS[name]
    lens = {"r0": 60, "r1": 41, "r2": 77, "r3": 1, "r4": 35, "r5": 52, "r6": 66, "r7": 2}
    reqs = {r: H.random_tokens(c["cfg"].vocab, n, i) for i, (r, n) in enumerate(lens.items())}
    pages = 192 // c["page"]                   # 192 tokens of cache for 334 tokens of eight requests, three at a time
    r = _runner(name, backend, "float32", pages, max_requests=3)
    got = H.run_mixed(r, reqs, seed=3, max_live=3)
    for rid, toks in reqs.items():
        assert K.err(got[rid], K.plain_logits(K.model_folder(name), toks)) < MODEL_TOL["float32"], rid
    assert all(pool.num_free == pages for pool in r.cache.pools)
    # each request alone gives what it gave in the batches
    alone = _runner(name, backend, "float32", pages, max_requests=1)
    for rid in ("r1", "r3", "r6"):
        one = H.run_portions(alone, rid, reqs[rid], [len(reqs[rid])])
        assert K.err(got[rid], one) < 1e-5, rid


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_residual_stream_after_every_layer(backend):
    """Layer by layer: the float32 stream after a layer is the plain implementation's.  The stream takes a layer's
    addends inside the norm that follows, so it is read where that norm leaves it."""
    name = "a"
    c = K.CONFIGS[name]
    toks = H.random_tokens(c["cfg"].vocab, 37, 9)
    cfg, w = K.plain_model(K.model_folder(name))
    _, streams = plain.forward(cfg, w, toks, return_layers=True)
    r = _runner(name, backend, "float32", 8)
    seen = []
    inner = r.kernels.stream_scaled_norm

    def spy(addends, residual, *a, **kw):
        out = inner(addends, residual, *a, **kw)
        seen.append(out[2].detach().float().cpu().clone())
        return out
    r.kernels.stream_scaled_norm = spy
    try:
        H.run_portions(r, "x", toks, [len(toks)])
    finally:
        del r.kernels.stream_scaled_norm
    # every layer's norms see the stream once (a layer without a feed-forward through its one norm, behind the first
    # layer), and the final norm
    assert len(seen) >= len(cfg["layers"])
    for i, want in enumerate(streams):
        assert float((seen[i + 1 - (len(cfg["layers"]) + 1 - len(seen))].double() - want).abs().max() / want.abs().max()) < 2e-5, i


# ------------------------------------------------------------------------------ the engine
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("schedule", ["prefill_first", "mixed"])
def test_greedy_generation_through_the_engine(backend, schedule):
    name = "d"
    c = K.CONFIGS[name]
    kernels, dev = _kernels(backend)
    folder = K.model_folder(name)
    prompts = [H.random_tokens(c["cfg"].vocab, n, 60 + n) for n in (3, 30, 1, 47, 18)]
    # few pages, three requests at a time and portions of at most 16 tokens: prompts are cut, requests wait
    llm = LLM(folder, kernels=kernels, device=dev, dtype="float32", kvcache_block_size=c["page"], num_kvcache_blocks=10,
              max_num_batched_tokens=16, max_num_seqs=3, schedule=schedule, max_model_len=128)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True), use_tqdm=False)
    cfg, w = K.plain_model(folder)
    for p, o in zip(prompts, outs):
        assert o["token_ids"] == plain.greedy_generate(cfg, w, p, 10), len(p)
    assert all(pool.num_free == 10 for pool in llm.runner.cache.pools)


@pytest.mark.gpu
def test_generation_in_bfloat16_with_captured_steps_and_bursts():
    name = "b"
    c = K.CONFIGS[name]
    folder = K.model_folder(name, "bfloat16")
    prompts = [H.random_tokens(c["cfg"].vocab, n, 80 + n) for n in (5, 40, 90, 17)]
    sp = SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True)
    common = dict(dtype="bfloat16", kvcache_block_size=c["page"], num_kvcache_blocks=24, max_num_seqs=4, max_model_len=256)
    eager = LLM(folder, enforce_eager=True, **common).generate(prompts, sp, use_tqdm=False)
    graphs = LLM(folder, decode_burst=8, **common)
    assert graphs.runner._graph_max_batch, "nothing in the model's single-token step asks the host: its steps are captured"
    fast = graphs.generate(prompts, sp, use_tqdm=False)
    for a, b in zip(eager, fast):
        assert a["token_ids"] == b["token_ids"]


@pytest.mark.gpu
def test_trace_replay_of_a_model_folder(tmp_path):
    """bin/trace_run as a process on a Pemuvik folder: portions, single tokens and a second request that takes the
    first one's pages."""
    import os
    import subprocess
    import sys
    import numpy as np
    name = "d"
    c = K.CONFIGS[name]
    folder = K.model_folder(name)
    a, b = H.random_tokens(c["cfg"].vocab, 50, 1), H.random_tokens(c["cfg"].vocab, 70, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:33], "want": [0, 32]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[33:34], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[34:], "want": [15]}, {"id": "b", "tokens": b[:2], "want": []}], "end": ["a"]},
             {"step": 3, "entries": [{"id": "b", "tokens": b[2:], "want": [67]}], "end": ["b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
                       timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    wa, wb = K.plain_logits(folder, a), K.plain_logits(folder, b)
    vocab = c["cfg"].vocab
    read = lambda i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, vocab))
    assert K.err(read(0), wa[[0, 32]]) < MODEL_TOL["float32"]
    assert K.err(read(1), wa[[33]]) < MODEL_TOL["float32"]
    assert K.err(read(2), wa[[49]]) < MODEL_TOL["float32"]
    assert K.err(read(3), wb[[69]]) < MODEL_TOL["float32"]
