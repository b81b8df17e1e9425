"""Nozurax: every mechanism alone, and the model through the step function and the engine, against
the plain implementation (tests/plain_nozurax.py).  Each test runs on the CPU stand-ins of the
device operations (tests/torch_kernels.py; this checks the stand-ins and the host logic) and, marked
gpu, on the HIP kernels."""
import math
import random
from types import SimpleNamespace

import pytest
import torch

import helpers as H
import nozurax_cases as N
import plain_nozurax as plain
from nano_vllm_amd import LLM, SamplingParams
from nano_vllm_amd.config import ConfigError, NozuraxConfig, architecture_of
from nano_vllm_amd.engine.batch import StepEntry
from nano_vllm_amd.engine.runner import ModelRunner
from torch_kernels import TorchKernels, new_caches

BACKENDS = ["cpu", pytest.param("hip", marks=pytest.mark.gpu)]
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


def _close(got, want, dtype, what=""):
    e = float((got.double().cpu() - want.double()).abs().max() / max(float(want.double().abs().max()), 1e-9))
    assert e < _tol(dtype), f"{what}: differs by {e:.2e} of the largest"


DTYPES = [torch.float32, torch.bfloat16]


# ------------------------------------------------------------------------------ configuration
def test_config_is_read_written_and_refused():
    cfg = N.CONFIGS["p"]["cfg"]
    d = cfg.to_dict()
    assert NozuraxConfig.from_dict(d) == cfg
    assert architecture_of(d).name == "Nozurax"
    spec = architecture_of(d).build_spec(cfg)
    # five entries, three layers with tensors: the entries that name another layer run its tensors again
    assert [r.layer for r in spec.order] == [0, 1, 0, 1, 2] and len(spec.layers) == 3
    assert all(r.cache_of is None for r in spec.order)
    assert "feed_forward" not in spec.layers[2].parts

    def broken(change):
        e = NozuraxConfig.from_dict(d).to_dict()
        change(e)
        with pytest.raises(ConfigError):
            NozuraxConfig.from_dict(e)
    broken(lambda e: e["layers"][0]["mixer"].__setitem__("decay", [0.5]))
    broken(lambda e: e["layers"][0]["mixer"]["rot"].__setitem__("dims", 7))
    broken(lambda e: e["layers"][1]["mixer"].__setitem__("kv_heads", 4))
    broken(lambda e: e["layers"][2].__setitem__("weights_of", 3))
    broken(lambda e: e["layers"][1]["mixer"]["q_temp"].__setitem__("every", 0))
    broken(lambda e: e["layers"][0].__setitem__("type", "convolution"))
    broken(lambda e: e["layers"][0]["mlp"].__setitem__("kind", "experts"))
    broken(lambda e: e.pop("norm"))


def test_the_checkpoint_is_read_by_its_own_names():
    from nano_vllm_amd.parts.model import Model
    from nano_vllm_amd.weights.loader import WeightError, checkpoint_layout, load_weights
    from safetensors.torch import load_file, save_file
    import os, shutil, tempfile
    folder = N.model_folder("p")
    cfg = N.CONFIGS["p"]["cfg"]
    spec = architecture_of(cfg.to_dict()).build_spec(cfg)
    model = Model(spec, TorchKernels(), "cpu")
    names = set(checkpoint_layout(model))
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.mix.g", "l1.mix.q.b", "l1.mix.k.norm", "l1.mix.sink",
            "l0.mlp.gate", "l4.mix.o"} <= names
    assert not any(n.startswith("l2.") or n.startswith("l3.") or n.startswith("l4.mlp") for n in names)
    assert set(load_file(os.path.join(folder, "model.safetensors"))) == names
    with tempfile.TemporaryDirectory() as tmp:
        shutil.copy(os.path.join(folder, "config.json"), tmp)
        t = load_file(os.path.join(folder, "model.safetensors"))
        t.pop("l1.mix.sink")
        t["l2.norm1"] = t["l0.norm1"].clone()
        save_file(t, os.path.join(tmp, "model.safetensors"))
        with pytest.raises(WeightError) as e:
            load_weights(Model(spec, TorchKernels(), "cpu"), tmp)
        assert e.value.missing == ["l1.mix.sink"] and e.value.unexpected == ["l2.norm1"]


# ------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_of_the_float_stream(backend, dtype):
    k, dev = _kernels(backend, dtype)
    g = torch.Generator().manual_seed(1)
    for rows, width in ((5, 48), (3, 333), (1, 2048), (2, 4100)):
        a = torch.randn((rows, width), generator=g).to(dtype)
        b = torch.randn((rows, width), generator=g).to(dtype)
        w = (0.3 * torch.randn(width, generator=g)).to(dtype)
        r0 = 30.0 * torch.randn((rows, width), generator=g)         # a stream that bfloat16 could not hold beside the addends
        r = r0.clone().to(dev)
        y, r2 = k.stream_rms_norm((a.to(dev), b.to(dev)), r, w.to(dev), 1e-5, 1.0)
        assert r2 is r and r.dtype == torch.float32
        want_r = r0.double() + (a.double() + b.double())
        _close(r, want_r, torch.float32, "stream")
        _close(y, plain.one_plus_norm(want_r, w.double(), 1e-5), dtype, "norm")
        # the stream starts with its one addend; a plain weight has offset 0
        y, r = k.stream_rms_norm((a.to(dev),), None, w.to(dev), 1e-5, 0.0)
        _close(r, a.double(), torch.float32, "first stream")
        _close(y, plain.unit_rms(a.double(), 1e-5) * w.double(), dtype, "first norm")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_gating_with_each_activation(backend, dtype):
    k, dev = _kernels(backend, dtype)
    g = torch.Generator().manual_seed(2)
    for rows, inner in ((4, 40), (3, 101)):
        x = (2.0 * torch.randn((rows, 2 * inner), generator=g)).to(dtype)
        a, u = x[:, :inner].double(), x[:, inner:].double()
        want = {"relu": torch.relu(a) * u, "silu": a * torch.sigmoid(a) * u,
                "gelu_tanh": 0.5 * a * (1 + torch.tanh(math.sqrt(2 / math.pi) * (a + 0.044715 * a ** 3))) * u}
        for act, w in want.items():
            _close(k.act_mul(x.to(dev), act), w, dtype, act)


@pytest.mark.gpu
@pytest.mark.parametrize("act", ["relu", "gelu_tanh", "silu"])
def test_gated_products_with_each_activation_at_every_row_count(act):
    # the product kernels gate in their epilogues: every kernel that a row count and a weight's shape
    # select, against the product and the gating done apart in float
    k, dev = _kernels("hip", torch.bfloat16)
    g = torch.Generator().manual_seed(11)
    for inner, width in ((96, 64), (1536, 512), (5120, 256)):
        w = (torch.randn((2 * inner, width), generator=g) / math.sqrt(width)).to(torch.bfloat16).to(dev)
        for rows in (1, 3, 8, 16, 40, 130, 256, 300):
            x = torch.randn((rows, width), generator=g).to(torch.bfloat16).to(dev)
            got = k.linear_act_mul(x, w, act)
            want = TorchKernels(dev, torch.bfloat16).linear_act_mul(x, w, act)
            _close(got, want.cpu(), torch.bfloat16, f"{act} inner {inner} rows {rows}")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,D,DV,page,every", [(6, 2, 16, 24, 8, 5), (4, 4, 24, 24, 16, 1), (3, 1, 40, 16, 4, 7)])
def test_whole_projection_norms_temperature_and_store(backend, dtype, hq, hkv, D, DV, page, every):
    k, dev = _kernels(backend, dtype)
    g = torch.Generator().manual_seed(3)
    # positions around the temperature's steps: floor((p + 1) / every) grows at p = every - 1, 2 every - 1, ...
    positions = sorted({0, 1, every - 2, every - 1, every, 2 * every - 1, 2 * every, 9 * every - 1, 9 * every, 300} - {-1})
    T = len(positions)
    qd, kd, vd = hq * D, hkv * D, hkv * DV
    qkv = (3.0 * torch.randn((T, qd + kd + vd), generator=g)).to(dtype)
    qw = (1.5 + 0.5 * torch.randn(qd, generator=g)).to(dtype)
    kw = (1.5 + 0.5 * torch.randn(kd, generator=g)).to(dtype)
    pages = 6
    kc, vc = new_caches(pages, hkv, D, page, dtype, dev, v_head_dim=DV)
    kc.fill_(float("nan")), vc.fill_(float("nan"))
    slots = random.Random(4).sample(range(pages * page), T)
    slots[2] = -1                                                   # a row that stores nothing
    x = qkv.clone().to(dev)
    q = k.qk_rownorm_store(x, hq, hkv, D, DV, qw.to(dev), kw.to(dev), 1e-6,
                           torch.tensor(positions, dtype=torch.int32, device=dev), 0.7, every,
                           torch.tensor(slots, dtype=torch.int32, device=dev), kc, vc)
    f = qkv.double()
    temp = torch.tensor([1 + 0.7 * math.log((p + 1) // every + 1) for p in positions], dtype=torch.float64)
    want_q = plain.unit_rms(f[:, :qd], 1e-6) * qw.double() * temp[:, None]
    want_k = plain.unit_rms(f[:, qd:qd + kd], 1e-6) * kw.double()
    _close(q, want_q, dtype, "q")
    vt = vc.shape[4]
    stored = 0
    for t, s in enumerate(slots):
        if s < 0:
            continue
        p, o = s // page, s % page
        _close(kc[p, :, o, :].reshape(-1), want_k[t], dtype, "stored k")
        _close(vc[p, :, o // vt, :, o % vt].reshape(-1), f[t, qd + kd:], dtype, "stored v")
        stored += 1
    assert int((~torch.isnan(kc.float())).sum()) == stored * kd and int((~torch.isnan(vc.float())).sum()) == stored * vd


def _sink_case(dtype, dev, hq, hkv, D, DV, page, lens, q_lens, seed, boost=None):
    """Requests with kv lengths `lens`, the last q_lens of which are this step's queries; keys and
    values scattered over shuffled pages (what unused slots hold must not matter: NaN)."""
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    S = len(lens)
    pages_per = [(n + page - 1) // page for n in lens]
    total = sum(pages_per) + 2
    order = list(range(total))
    rng.shuffle(order)
    kc, vc = new_caches(total, hkv, D, page, dtype, dev, v_head_dim=DV)
    kc.fill_(float("nan")), vc.fill_(float("nan"))
    vt = vc.shape[4]
    tables = torch.full((S, max(pages_per)), -1, dtype=torch.int32)
    ks, vs, qs, token_seq, positions = [], [], [], [], []
    for s, n in enumerate(lens):
        mine = [order.pop() for _ in range(pages_per[s])]
        tables[s, : len(mine)] = torch.tensor(mine, dtype=torch.int32)
        kk = torch.randn((n, hkv, D), generator=g).to(dtype)
        vv = torch.randn((n, hkv, DV), generator=g).to(dtype)
        qq = torch.randn((n, hq, D), generator=g).to(dtype)
        if boost is not None:               # one key that every query prefers by far
            kk[boost] = 0
            kk[boost, :, 0] = 8.0
            qq[:] = 0
            qq[:, :, 0] = 8.0
        for j in range(n):
            kc[mine[j // page], :, j % page, :] = kk[j].to(dev)
            vc[mine[j // page], :, (j % page) // vt, :, (j % page) % vt] = vv[j].to(dev)
        ks.append(kk), vs.append(vv), qs.append(qq)
        token_seq += [s] * q_lens[s]
        positions += list(range(n - q_lens[s], n))
    q = torch.cat([qs[s][lens[s] - q_lens[s]:] for s in range(S)]).reshape(sum(q_lens), hq * D).contiguous().to(dev)
    order_ok = all(a == 1 or b != 1 for a, b in zip(q_lens, q_lens[1:]))
    assert order_ok, "single tokens come first in a batch"
    batch = SimpleNamespace(
        num_seqs=S, num_tokens=sum(q_lens), token_seq=torch.tensor(token_seq, dtype=torch.int32, device=dev),
        positions=torch.tensor(positions, dtype=torch.int32, device=dev), max_kv_len=max(lens), max_q_len=max(q_lens),
        kv_lens=torch.tensor(lens, dtype=torch.int32, device=dev),
        cu_seqlens_q=torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32, device=dev),
        num_decode=next((i for i, n in enumerate(q_lens) if n != 1), len(q_lens)), q_lens=list(q_lens),
        starts=[n - m for n, m in zip(lens, q_lens)],
        groups=[SimpleNamespace(block_tables=tables.to(dev), slot_mapping=None)])
    return q, kc, vc, batch, (qs, ks, vs)


def _sink_softmax(qs, ks, vs, lens, q_lens, scale, sinks):
    """Dense, in double: the sink is one more term of the denominator and has no value."""
    rows = []
    for q, k, v, n, m in zip(qs, ks, vs, lens, q_lens):
        hq, hkv = q.shape[1], k.shape[1]
        for i in range(n - m, n):
            heads = []
            for h in range(hq):
                s = (k[: i + 1, h // (hq // hkv)].double() @ q[i, h].double()) * scale
                top = max(float(s.max()), float(sinks[h]))
                e = torch.exp(s - top)
                heads.append((e[:, None] * v[: i + 1, h // (hq // hkv)].double()).sum(0) /
                             (e.sum() + math.exp(float(sinks[h]) - top)))
            rows.append(torch.cat(heads))
    return torch.stack(rows)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,D,DV,page,lens,q_lens", [
    (6, 2, 16, 24, 8, [1, 9, 70, 33], [1, 1, 1, 1]),            # single tokens, the first of a sequence among them
    (4, 4, 24, 24, 16, [64, 65, 130], [64, 2, 41]),             # portions that end at, and just after, a page's border
    (3, 1, 40, 16, 4, [17, 5, 90], [1, 5, 37]),                 # mixed
    (8, 2, 64, 64, 32, [300, 96], [1, 96]),                     # equal head sizes
])
def test_attention_with_sinks_and_values_of_their_own_size(backend, dtype, hq, hkv, D, DV, page, lens, q_lens):
    k, dev = _kernels(backend, dtype)
    q, kc, vc, batch, (qs, ks, vs) = _sink_case(dtype, dev, hq, hkv, D, DV, page, lens, q_lens, seed=5)
    for sinks in (torch.linspace(-1.0, 3.0, hq), torch.full((hq,), -60.0), torch.full((hq,), 40.0)):
        got = k.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, 0.3, None, v_head_dim=DV, sinks=sinks.to(dev))
        assert tuple(got.shape) == (sum(q_lens), hq * DV)
        want = _sink_softmax(qs, ks, vs, lens, q_lens, 0.3, sinks)
        e = float((got.double().cpu() - want).abs().max())
        assert e < (2e-5 if dtype == torch.float32 else 3e-2), (sinks[0], e)
    # a sink far below every score is no sink; one far above takes every weight
    none = k.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, 0.3, None, v_head_dim=DV).float().cpu()
    assert float((none.double() - _sink_softmax(qs, ks, vs, lens, q_lens, 0.3, torch.full((hq,), -60.0))).abs().max()) < 3e-2
    assert float(got.float().abs().max()) < 1e-6
    if hasattr(k, "check_faults"):
        k.check_faults()


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_with_a_sink_reads_a_far_key_among_hundreds(backend, dtype):
    k, dev = _kernels(backend, dtype)
    hq, hkv, D, DV, page = 4, 2, 32, 48, 16
    for lens, q_lens in (([600], [40]), ([600], [1])):
        q, kc, vc, batch, (qs, ks, vs) = _sink_case(dtype, dev, hq, hkv, D, DV, page, lens, q_lens, seed=6, boost=3)
        # key 3 scores 64, the sink 60: the output is e^4 / (e^4 + 1) of key 3's value
        got = k.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, 1.0, None, v_head_dim=DV,
                                sinks=torch.full((hq,), 60.0, device=dev)).float().cpu()
        share = math.exp(4) / (math.exp(4) + 1)
        want = share * vs[0][3].float().repeat_interleave(hq // hkv, 0).reshape(1, hq * DV).expand(q_lens[0], -1)
        assert float((got - want).abs().max()) < 0.05


@pytest.mark.gpu
def test_sinks_in_the_matrix_core_kernels_over_long_contexts():
    # single tokens whose keys are shared out over many waves and merged, and a long portion: the
    # matrix-core kernels against the general ones, and both against the dense softmax
    k, dev = _kernels("hip", torch.bfloat16)
    hq, hkv, D, page = 8, 2, 128, 64
    lens, q_lens = [3000, 5000, 700], [1, 1, 260]
    q, kc, vc, batch, (qs, ks, vs) = _sink_case(torch.bfloat16, dev, hq, hkv, D, D, page, lens, q_lens, seed=9)
    sinks = torch.linspace(-2.0, 6.0, hq)
    fast = k.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, D ** -0.5, None, v_head_dim=D, sinks=sinks.to(dev)).float().cpu()
    k.mfma_attention = False
    try:
        general = k.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, D ** -0.5, None, v_head_dim=D, sinks=sinks.to(dev)).float().cpu()
    finally:
        k.mfma_attention = True
    want = _sink_softmax(qs, ks, vs, lens, q_lens, D ** -0.5, sinks)
    assert float((general.double() - want).abs().max()) < 1e-2
    assert float((fast.double() - want).abs().max()) < 2e-2
    # the sink's share is visible: without it the outputs are larger
    none = k.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, D ** -0.5, None).float().cpu()
    assert float((none - fast).abs().max()) > 5e-3
    k.check_faults()


def _retention_inputs(heads, dim, vdim, T, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    hidden = heads * vdim
    h = torch.randn((T, hidden), generator=g, dtype=torch.float64)
    w = {n: torch.randn((heads * d, hidden), generator=g, dtype=torch.float64) / math.sqrt(hidden)
         for n, d in (("q", dim), ("k", dim), ("v", vdim), ("g", vdim))}
    proj = torch.cat([h @ w[n].T for n in ("q", "k", "v", "g")], dim=1).to(dtype)
    return proj


def _plain_retention_of_projections(proj, heads, dim, vdim, decay, rot, base, eps):
    """plain.retention on projections that are given: the input is the projections' row and the
    weights pick its parts out."""
    width = proj.shape[1]
    eye = torch.eye(width, dtype=torch.float64)
    qk, vv = heads * dim, heads * vdim
    w = {"q": eye[:qk], "k": eye[qk:2 * qk], "v": eye[2 * qk:2 * qk + vv], "g": eye[2 * qk + vv:], "o": torch.eye(vv, dtype=torch.float64)}
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot:
        m["rot"] = {"dims": rot, "base": base}
    return plain.retention(proj.double(), w, "", m, eps, torch.arange(proj.shape[0]))


def _state_batch(dev, q_lens, starts, slots):
    return SimpleNamespace(
        num_seqs=len(q_lens), q_lens=list(q_lens), starts=list(starts),
        num_decode=next((i for i, n in enumerate(q_lens) if n != 1), len(q_lens)),
        positions=torch.tensor([p for s, n in zip(starts, q_lens) for p in range(s, s + n)], dtype=torch.int32, device=dev),
        cu_seqlens_q=torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32, device=dev),
        seq_starts=torch.tensor(starts, dtype=torch.int32, device=dev),
        state_slots=torch.tensor(slots, dtype=torch.int32, device=dev))


def _retention_constants(k, dev, decay, dim, rot, base):
    chunk = k.RETENTION_CHUNK
    powers = (torch.tensor(decay, dtype=torch.float64)[:, None] ** torch.arange(chunk + 1, dtype=torch.float64)[None, :])
    inv_freq = None
    if rot:
        inv_freq = (base ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / rot)).float().to(dev)
    return powers.float().contiguous().to(dev), inv_freq


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim,decay,rot,base", [
    (3, 16, 8, (0.5, 0.9, 0.999), 8, 100.0),
    (1, 32, 32, (0.9375,), 32, 1e6),
    (2, 24, 40, (0.97, 1.0), 0, 0.0),
    (2, 64, 72, (0.95, 0.998), 64, 1e4),
    (2, 6, 10, (0.0, 0.99), 4, 50.0),
    # heads and values of multiples of 32 channels: the kernel on the matrix cores
    (2, 64, 64, (0.93, 0.9975), 64, 1e4),
    (2, 128, 160, (0.9, 0.999), 64, 1e6),
    (1, 256, 32, (0.99,), 0, 0.0),
    (3, 96, 96, (0.5, 1.0, 0.75), 96, 100.0),
    (2, 32, 64, (0.9, 0.99), 8, 100.0),         # a rotation too narrow for the loads of eight elements
])
def test_retention_in_portions_of_every_size_and_token_by_token(backend, dtype, heads, dim, vdim, decay, rot, base):
    k, dev = _kernels(backend, dtype)
    T = 150
    proj = _retention_inputs(heads, dim, vdim, T, 7, dtype)
    want = _plain_retention_of_projections(proj, heads, dim, vdim, decay, rot, base, 1e-5)
    powers, inv_freq = _retention_constants(k, dev, decay, dim, rot, base)
    C = k.RETENTION_CHUNK
    cuts = [[T], [1] * 40 + [T - 40], [C - 1, 1, 1, C, C + 1, 2, T - 3 * C - 4], [2] * 20 + [T - 40], [3 * C, T - 3 * C]]
    for portions in cuts:
        # the slot holds what another request left there: a start at 0 must not read it
        state = torch.full((3, heads, dim, vdim), float("nan"), dtype=torch.float32, device=dev)
        got, pos = [], 0
        for n in portions:
            batch = _state_batch(dev, [n], [pos], [1])
            got.append(k.retention(proj[pos:pos + n].contiguous().to(dev), heads, dim, vdim, state, powers, inv_freq,
                                   dim ** -0.5, 1e-5, batch).float().cpu())
            pos += n
        e = float((torch.cat(got).double() - want).abs().max() / want.abs().max())
        assert e < (3e-5 if dtype == torch.float32 else 2e-2), (portions[:4], e)
        assert bool(torch.isnan(state[0]).all()) and bool(torch.isnan(state[2]).all()) and not bool(torch.isnan(state[1]).any())


@pytest.mark.parametrize("backend", BACKENDS)
def test_retention_of_unequal_requests_in_one_batch(backend):
    dtype = torch.float32
    k, dev = _kernels(backend, dtype)
    heads, dim, vdim, decay, rot, base = 3, 16, 24, (0.5, 0.95, 1.0), 16, 1e4
    powers, inv_freq = _retention_constants(k, dev, decay, dim, rot, base)
    lens = [70, 1, 33, 101]
    projs = [_retention_inputs(heads, dim, vdim, n, 10 + i, dtype) for i, n in enumerate(lens)]
    wants = [_plain_retention_of_projections(p, heads, dim, vdim, decay, rot, base, 1e-6) for p in projs]
    state = torch.full((5, heads, dim, vdim), float("nan"), dtype=torch.float32, device=dev)
    slots = [3, 0, 4, 1]
    # step 1: request 1 whole (one token, comes first), portions of the others; step 2: the rest
    first = [40, 1, 32, 2]
    order = [1, 0, 2, 3]
    x = torch.cat([projs[i][: first[i]] for i in order]).to(dev)
    batch = _state_batch(dev, [first[i] for i in order], [0] * 4, [slots[i] for i in order])
    got1 = k.retention(x, heads, dim, vdim, state, powers, inv_freq, dim ** -0.5, 1e-6, batch).float().cpu()
    rest = [0, 2, 3]
    x = torch.cat([projs[i][first[i]:] for i in rest]).to(dev)
    batch = _state_batch(dev, [lens[i] - first[i] for i in rest], [first[i] for i in rest], [slots[i] for i in rest])
    got2 = k.retention(x, heads, dim, vdim, state, powers, inv_freq, dim ** -0.5, 1e-6, batch).float().cpu()
    at1, at2 = 0, 0
    for i in order:
        got = got1[at1:at1 + first[i]]
        at1 += first[i]
        if i in rest:
            got = torch.cat((got, got2[at2:at2 + lens[i] - first[i]]))
            at2 += lens[i] - first[i]
        assert float((got.double() - wants[i]).abs().max() / wants[i].abs().max()) < 3e-5, i
    assert bool(torch.isnan(state[2]).all())                         # the slot that no request holds


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_retention_of_long_portions_whose_blocks_run_side_by_side(dtype):
    # portions of many blocks beside a short one and one that continues a state; with the blocks one
    # after the other the same numbers but for rounding
    k, dev = _kernels("hip", dtype)
    heads, dim, vdim, decay, rot, base = 2, 64, 96, (0.9, 0.9995), 32, 1e4
    powers, inv_freq = _retention_constants(k, dev, decay, dim, rot, base)
    lens = [700, 40, 333]
    first = [0, 0, 100]                       # request 2 has 100 tokens in its state already
    projs = [_retention_inputs(heads, dim, vdim, n, 30 + i, dtype) for i, n in enumerate(lens)]
    wants = [_plain_retention_of_projections(p, heads, dim, vdim, decay, rot, base, 1e-6) for p in projs]
    results = {}
    for side_by_side in (True, False):
        k.retention_blocks_side_by_side = side_by_side
        try:
            state = torch.full((3, heads, dim, vdim), float("nan"), dtype=torch.float32, device=dev)
            k.retention(projs[2][:100].contiguous().to(dev), heads, dim, vdim, state, powers, inv_freq, dim ** -0.5, 1e-6,
                        _state_batch(dev, [100], [0], [2]))
            x = torch.cat([p[f:] for p, f in zip(projs, first)]).to(dev)
            batch = _state_batch(dev, [n - f for n, f in zip(lens, first)], first, [0, 1, 2])
            got = k.retention(x, heads, dim, vdim, state, powers, inv_freq, dim ** -0.5, 1e-6, batch).float().cpu()
            results[side_by_side] = (got, state.clone())
        finally:
            k.retention_blocks_side_by_side = True
        at = 0
        for want, f in zip(wants, first):
            n = want.shape[0] - f
            e = float((got[at:at + n].double() - want[f:]).abs().max() / want.abs().max())
            assert e < (3e-5 if dtype == torch.float32 else 2e-2), (side_by_side, e)
            at += n
    assert float((results[True][0] - results[False][0]).abs().max()) < (1e-4 if dtype == torch.float32 else 5e-2)
    a, b = results[True][1], results[False][1]
    assert float((a - b).abs().max() / b.abs().max()) < 1e-5          # the states the requests are left with


@pytest.mark.parametrize("backend", BACKENDS)
def test_retention_keeps_a_far_token_by_its_decay(backend):
    # token 0 carries a large key and value; a query like its key stands 400 tokens later: the head
    # that does not decay still reads it in full, the head that halves every token reads nothing of it
    k, dev = _kernels(backend, torch.float32)
    heads, dim, vdim, T = 2, 8, 4, 401
    proj = torch.zeros((T, 2 * heads * (dim + vdim)))
    qk, vv = heads * dim, heads * vdim
    g = torch.Generator().manual_seed(8)
    proj[:, qk:2 * qk] = 0.01 * torch.randn((T, qk), generator=g)
    proj[:, 2 * qk:2 * qk + vv] = 0.01 * torch.randn((T, vv), generator=g)
    proj[:, 2 * qk + vv:] = 1.0
    for h in range(heads):
        proj[0, qk + h * dim] = 10.0                      # k_0
        proj[0, 2 * qk + h * vdim + 1] = 10.0             # v_0
        proj[T - 1, h * dim] = 10.0                       # q_400
    powers, inv_freq = _retention_constants(k, dev, (1.0, 0.5), dim, 0, 0.0)
    state = torch.zeros((1, heads, dim, vdim), dtype=torch.float32, device=dev)
    for portions in ([T], [T - 1, 1]):
        pos, out = 0, None
        for n in portions:
            out = k.retention(proj[pos:pos + n].contiguous().to(dev), heads, dim, vdim, state, powers, inv_freq, 1.0, 1e-6,
                              _state_batch(dev, [n], [pos], [0])).float().cpu()
            pos += n
        y = out[-1].reshape(heads, vdim)
        # head 0: o is 1000 at channel 1 and small elsewhere, so o / rms(o) is 2 there (4 channels); times silu(1)
        assert abs(float(y[0, 1]) - 2.0 * (1 / (1 + math.exp(-1)))) < 1e-2
        assert float(y[1].abs().max()) < 1.9 and abs(float(y[1, 1])) < 1.5   # head 1 has forgotten token 0


# ------------------------------------------------------------------------------ the model, through the step function
def _runner(name, backend, dtype, pages, max_requests=4):
    kernels, dev = _kernels(backend, torch.float32 if dtype == "float32" else torch.bfloat16)
    return H.make_runner(N.model_folder(name, dtype), dtype, N.CONFIGS[name]["page"], pages, device=dev,
                         kernels=kernels, max_requests=max_requests)


MODEL_TOL = {"float32": 1e-4, "bfloat16": 6e-2}


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["p", "q", "r", "s"])
def test_every_cutting_gives_the_plain_logits(backend, name):
    c = N.CONFIGS[name]
    n = 110
    toks = H.random_tokens(c["cfg"].vocab, n, 1)
    want = N.plain_logits(N.model_folder(name), toks)
    r = _runner(name, backend, "float32", 40)
    for portions in (H.whole(n), H.last_one_by_one(n, 45), H.changing_portions(n, 2), [1] * 3 + [2] * 10 + [n - 23]):
        got = H.run_portions(r, "x", toks, portions)
        assert N.err(got, want) < MODEL_TOL["float32"], portions


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["p", "r"])
def test_bfloat16_follows_the_plain_logits_under_every_cutting(name):
    c = N.CONFIGS[name]
    n = 130
    toks = H.random_tokens(c["cfg"].vocab, n, 3)
    want = N.plain_logits(N.model_folder(name, "bfloat16"), toks)
    r = _runner(name, "hip", "bfloat16", 40)
    for portions in (H.whole(n), H.last_one_by_one(n, 40), H.changing_portions(n, 4)):
        got = H.run_portions(r, "x", toks, portions)
        assert N.err(got, want) < MODEL_TOL["bfloat16"], portions


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_first_tokens_of_a_sequence(backend):
    c = N.CONFIGS["q"]
    r = _runner("q", backend, "float32", 8)
    for n in (1, 2, 3):
        toks = H.random_tokens(c["cfg"].vocab, n, 40 + n)
        want = N.plain_logits(N.model_folder("q"), toks)
        for portions in ([n], [1] * n):
            assert N.err(H.run_portions(r, "x", toks, portions), want) < MODEL_TOL["float32"], (n, portions)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["p", "s"])
def test_long_decoding(backend, name):
    # one prompt token, then 170 tokens one by one: over pages, chunks and steps of the temperature
    c = N.CONFIGS[name]
    n = 171
    toks = H.random_tokens(c["cfg"].vocab, n, 5)
    want = N.plain_logits(N.model_folder(name), toks)
    r = _runner(name, backend, "float32", 48)
    assert N.err(H.run_portions(r, "x", toks, [1] * n), want) < MODEL_TOL["float32"]


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["p", "q"])
def test_mixed_batches_on_pages_and_slots_that_are_used_again(backend, name):
    c = N.CONFIGS[name]
    lens = {"r0": 60, "r1": 41, "r2": 77, "r3": 1, "r4": 35, "r5": 52, "r6": 66, "r7": 2}
    reqs = {r: H.random_tokens(c["cfg"].vocab, n, i) for i, (r, n) in enumerate(lens.items())}
    pages = 180 // c["page"]                   # 180 tokens of cache and three state slots for 334 tokens of eight requests
    r = _runner(name, backend, "float32", pages, max_requests=3)
    got = H.run_mixed(r, reqs, seed=3, max_live=3)
    for rid, toks in reqs.items():
        assert N.err(got[rid], N.plain_logits(N.model_folder(name), toks)) < MODEL_TOL["float32"], rid
    assert r.cache.pools[0].num_free == pages and r.cache.slots.num_free == 3
    # each request alone gives what it gave in the batches
    alone = _runner(name, backend, "float32", pages, max_requests=1)
    for rid in ("r1", "r3", "r6"):
        one = H.run_portions(alone, rid, reqs[rid], [len(reqs[rid])])
        assert N.err(got[rid], one) < 1e-5, rid


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_residual_stream_after_every_layer(backend):
    """Layer by layer: the float32 stream that each norm is handed is the plain implementation's."""
    name = "p"
    c = N.CONFIGS[name]
    toks = H.random_tokens(c["cfg"].vocab, 37, 9)
    cfg, w = N.plain_model(N.model_folder(name))
    _, streams = plain.forward(cfg, w, toks, return_layers=True)
    r = _runner(name, backend, "float32", 8)
    seen = []
    inner = r.kernels.stream_rms_norm

    def spy(addends, residual, *a, **kw):
        y, res = inner(addends, residual, *a, **kw)
        seen.append(res.detach().float().cpu().clone())
        return y, res
    r.kernels.stream_rms_norm = spy
    try:
        H.run_portions(r, "x", toks, [len(toks)])
    finally:
        del r.kernels.stream_rms_norm
    assert len(seen) == len(cfg["layers"]) + 1                      # the embedding, then the stream after every layer
    for i, want in enumerate(streams):
        assert float((seen[i + 1].double() - want).abs().max() / want.abs().max()) < 2e-5, i


# ------------------------------------------------------------------------------ the engine
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("schedule", ["prefill_first", "mixed"])
def test_greedy_generation_through_the_engine(backend, schedule):
    name = "q"
    c = N.CONFIGS[name]
    kernels, dev = _kernels(backend)
    folder = N.model_folder(name)
    prompts = [H.random_tokens(c["cfg"].vocab, n, 60 + n) for n in (3, 30, 1, 47, 18)]
    # few pages, three request slots and portions of at most 16 tokens: prompts are cut, requests wait
    llm = LLM(folder, kernels=kernels, device=dev, dtype="float32", kvcache_block_size=c["page"], num_kvcache_blocks=10,
              max_num_batched_tokens=16, max_num_seqs=3, schedule=schedule, max_model_len=128)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True), use_tqdm=False)
    cfg, w = N.plain_model(folder)
    for p, o in zip(prompts, outs):
        assert o["token_ids"] == plain.greedy_generate(cfg, w, p, 12), len(p)
    assert llm.runner.cache.slots.num_free == 3 and llm.runner.cache.pools[0].num_free == 10


@pytest.mark.parametrize("backend", BACKENDS)
def test_models_of_one_kind_of_layer_and_tensors_owned_by_a_later_layer(backend, tmp_path):
    # retention only (no pages at all), attention only (no state slots), and an entry that runs the
    # tensors of a layer further down the list; layers without a feed-forward among them
    from nano_vllm_amd.weights import write_random_model
    cases = {
        "retention": NozuraxConfig(vocab=120, width=40, eps=1e-6, layers=(
            N._ret(0, 2, 8, 12, (0.9, 0.99), rot=8, base=1e4, ff=None), N._ret(1, 1, 16, 8, (0.95,), ff=56))),
        "attention": NozuraxConfig(vocab=120, width=40, eps=1e-6, layers=(
            N._att(0, 4, 1, 8, 12, 0.3, ff=None), N._att(1, 2, 2, 16, 8, 0.2, coef=0.4, every=2, ff=48))),
        "later": NozuraxConfig(vocab=90, width=24, eps=1e-5, layers=(
            N._ret(0, 2, 8, 4, (0.9, 0.99), rot=4, base=10.0, ff=32, of=2), N._att(1, 2, 1, 8, 4, 0.3, coef=0.4, every=2, ff=None),
            N._ret(2, 2, 8, 4, (0.9, 0.99), rot=4, base=10.0, ff=32))),
    }
    kernels, dev = _kernels(backend)
    for name, cfg in cases.items():
        folder = write_random_model(str(tmp_path / name), cfg, seed=3, std=0.2, dtype="float32")
        c, w = plain.read_folder(folder)
        prompts = [H.random_tokens(cfg.vocab, n, 5 + n) for n in (1, 19, 40)]
        llm = LLM(folder, kernels=kernels, device=dev, dtype="float32", kvcache_block_size=8, num_kvcache_blocks=12,
                  max_num_batched_tokens=16, max_num_seqs=2, schedule="mixed", max_model_len=96)
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True), use_tqdm=False)
        for p, o in zip(prompts, outs):
            assert o["token_ids"] == plain.greedy_generate(c, w, p, 8), (name, len(p))


@pytest.mark.gpu
def test_generation_in_bfloat16_with_captured_steps_and_bursts():
    name = "r"
    c = N.CONFIGS[name]
    folder = N.model_folder(name, "bfloat16")
    prompts = [H.random_tokens(c["cfg"].vocab, n, 80 + n) for n in (5, 40, 90, 17)]
    sp = SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True)
    common = dict(dtype="bfloat16", kvcache_block_size=c["page"], num_kvcache_blocks=24, max_num_seqs=4, max_model_len=256)
    eager = LLM(folder, enforce_eager=True, **common).generate(prompts, sp, use_tqdm=False)
    graphs = LLM(folder, decode_burst=8, **common)
    assert graphs.runner._graph_max_batch, "a model with retention state is captured: its steps read the metadata on the device"
    fast = graphs.generate(prompts, sp, use_tqdm=False)
    for a, b in zip(eager, fast):
        assert a["token_ids"] == b["token_ids"]
    # and both follow the plain implementation until bfloat16 flips a near tie
    cfg, w = N.plain_model(folder)
    agree = total = 0
    for p, o in zip(prompts, fast):
        want = plain.greedy_generate(cfg, w, p, 12)
        total += len(want)
        agree += sum(int(a == b) for a, b in zip(o["token_ids"], want))
    assert agree >= 0.7 * total, (agree, total)
