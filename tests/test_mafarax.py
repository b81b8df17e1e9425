"""Mafarax: every mechanism alone, and the model through the step function and the engine, against
the plain implementation (tests/plain_mafarax.py).  Each test runs on the CPU stand-ins of the
device operations (tests/torch_kernels.py; this checks the stand-ins and the host logic) and, marked
gpu, on the HIP kernels."""
import json
import math
import random
from types import SimpleNamespace

import pytest
import torch

import helpers as H
import mafarax_cases as M
import plain_mafarax as plain
from nano_vllm_amd import LLM, SamplingParams
from nano_vllm_amd.config import ConfigError, MafaraxConfig, architecture_of
from nano_vllm_amd.engine.batch import StepEntry
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
    for c in M.CONFIGS.values():
        d = c["cfg"].to_dict()
        assert architecture_of(d).name == "Mafarax"
        assert MafaraxConfig.from_dict(json.loads(json.dumps(d))) == c["cfg"]
    d = M.CONFIGS["a"]["cfg"].to_dict()

    def broken(change):
        e = json.loads(json.dumps(d))
        change(e)
        with pytest.raises(ConfigError):
            MafaraxConfig.from_dict(e)
    broken(lambda e: e["layers"][0].update(type="serial"))
    broken(lambda e: e["layers"][0]["mixer"]["left"].update(kv_heads=3))
    broken(lambda e: e["layers"][0]["mixer"]["left"]["mask"].update(size=0))
    broken(lambda e: e["layers"][0]["mixer"]["left"]["rot"].update(dims=7))
    broken(lambda e: e["layers"][0]["mixer"]["right"].update(groups=2))
    broken(lambda e: e["layers"][0]["mlp"]["router"].update(top=5))
    broken(lambda e: e["layers"][0]["mlp"].update(kind="dense"))
    broken(lambda e: e.pop("width"))
    # what a configuration may leave out: the scaling (factor 1), the rotation, the groups, the shared expert
    e = json.loads(json.dumps(d))
    e["layers"][0]["mixer"]["left"]["rot"].pop("scaling")
    e["layers"][1]["mixer"]["left"].pop("rot")
    e["layers"][0]["mlp"]["router"].pop("groups")
    e["layers"][0]["mlp"].pop("shared")
    cfg = MafaraxConfig.from_dict(e)
    assert cfg.layers[0].left.rot_factor == 1.0 and cfg.layers[1].left.rot_dims == 0
    assert cfg.layers[0].mlp.group_count == 1 and cfg.layers[0].mlp.shared_ff is None


def test_the_checkpoint_is_read_by_its_own_names():
    from safetensors import safe_open
    folder = M.model_folder("a")
    with safe_open(folder + "/model.safetensors", "pt", "cpu") as f:
        names = set(f.keys())
    for want in ("embed", "head", "final.norm", "final.norm.b", "final.norm.alpha", "l0.norm1", "l0.norm2.alpha",
                 "l0.mix.left.q", "l0.mix.left.q.b", "l0.mix.left.o.b", "l0.mix.left.out", "l0.mix.right.out",
                 "l0.mix.right.in", "l0.mix.right.conv", "l0.mix.right.conv.b", "l0.mix.right.dt_bias",
                 "l0.mix.right.A_log", "l0.mix.right.D", "l0.mix.right.norm", "l0.mix.right.o", "l0.mlp.router",
                 "l0.mlp.e0.up", "l0.mlp.e5.down", "l0.mlp.shared.up", "l2.mlp.e3.up"):
        assert want in names, want
    assert not any(n.startswith("l1.mlp") or n.startswith("l1.norm2") or n.startswith("l2.mlp.shared") for n in names)
    assert "l0.mix.right.o.b" not in names


# ------------------------------------------------------------------------------ norms
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_dynamic_tanh_on_the_float_stream(backend, dtype):
    k, dev = _kernels(backend, dtype)
    g = torch.Generator().manual_seed(1)
    for rows, width in ((1, 20), (7, 48), (70, 300)):
        w, b = torch.randn(width, generator=g), torch.randn(width, generator=g)
        alpha = torch.tensor(0.8)
        a = (torch.randn((rows, width), generator=g) * 2).to(dtype)
        c = (torch.randn((rows, width), generator=g) * 2).to(dtype)
        y, r = k.stream_dyt((a.to(dev),), None, w.to(dev), b.to(dev), alpha.to(dev))
        assert r.dtype == torch.float32 and torch.equal(r.cpu(), a.float())
        _close(y, torch.tanh(0.8 * a.double()) * w.double() + b.double(), dtype, "first")
        y, r2 = k.stream_dyt((c.to(dev),), r, w.to(dev), b.to(dev), alpha.to(dev))
        assert r2.data_ptr() == r.data_ptr()
        want_r = a.double() + c.double()
        _close(r2, want_r, torch.float32, "stream")
        _close(y, torch.tanh(0.8 * want_r) * w.double() + b.double(), dtype, "second")
        # a stream far beyond bfloat16's grain keeps its small addends
        big = torch.full((rows, width), 300.0)
        _, r3 = k.stream_dyt((big.to(dtype).to(dev),), None, w.to(dev), b.to(dev), alpha.to(dev))
        _, r3 = k.stream_dyt((torch.full((rows, width), 0.25).to(dtype).to(dev),), r3, w.to(dev), b.to(dev), alpha.to(dev))
        assert torch.equal(r3.cpu(), torch.full((rows, width), 300.25))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_two_normed_halves_averaged(backend, dtype):
    k, dev = _kernels(backend, dtype)
    g = torch.Generator().manual_seed(2)
    for rows, width, eps in ((1, 20, 1e-5), (9, 72, 1e-6), (40, 520, 1e-6)):
        a = (torch.randn((rows, width), generator=g) * 3).to(dtype)
        b = (torch.randn((rows, width), generator=g) * 0.01).to(dtype)       # halves of very different size weigh alike
        wa, wb = torch.randn(width, generator=g), torch.randn(width, generator=g)
        got = k.pair_norm_mean(a.to(dev), wa.to(dev), b.to(dev), wb.to(dev), eps)
        want = 0.5 * (plain.unit(a.double(), eps) * wa.double() + plain.unit(b.double(), eps) * wb.double())
        _close(got, want, dtype, (rows, width))


# ------------------------------------------------------------------------------ rotation and store
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,D,DV,R,page,factor", [(4, 2, 16, 24, 8, 8, 4.0), (2, 2, 24, 8, 24, 4, 1.0), (3, 1, 10, 10, 6, 16, 1.5)])
def test_rotation_of_a_part_of_the_head_and_store(backend, dtype, hq, hkv, D, DV, R, page, factor):
    k, dev = _kernels(backend, dtype)
    g = torch.Generator().manual_seed(3)
    positions = [0, 1, 2, 5, 63, 64, 1000, 4097, 30000]
    T = len(positions)
    width = hq * D + hkv * D + hkv * DV
    qkv = torch.randn((T, width), generator=g).to(dtype)
    base = 500.0
    inv_freq = (1.0 / (base ** (torch.arange(0, R, 2, dtype=torch.float) / R)) / factor).to(dev)
    pos = torch.tensor(positions, dtype=torch.int32, device=dev)
    table = k.rotary_step_table(inv_freq, pos)
    want_angles = torch.tensor(positions, dtype=torch.float64)[:, None] * inv_freq.double().cpu()[None, :]
    assert float((table.cpu().double() - torch.cat((want_angles.cos(), want_angles.sin()), -1)).abs().max()) < 3e-3
    kc, vc = new_caches(3, hkv, D, page, dtype, dev, v_head_dim=DV)
    slots = torch.tensor([5, 0, 2 * page + 1, -1, page, 3, 1, 2, 2 * page + 2][:T], dtype=torch.int32, device=dev)
    q = k.qk_rownorm_store(qkv.clone().to(dev), hq, hkv, D, DV, None, None, 1e-6, pos, 0.0, 1, slots, kc, vc, rot_table=table)
    rot = {"dims": R, "base": base, "scaling": {"factor": factor}}

    def turned(x, heads):
        x = x.double().reshape(T, heads, D)
        return torch.stack([_turn_at(x[i], rot, p) for i, p in enumerate(positions)])
    want_q = turned(qkv[:, : hq * D], hq)
    tol = 2e-2 if dtype == torch.bfloat16 else 2e-3       # float angles of large positions
    _close(q.reshape(T, hq, D), want_q, dtype, "q", tol)
    want_k = turned(qkv[:, hq * D: hq * D + hkv * D], hkv)
    vt = vc.shape[4]
    for i, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        _close(kc[s // page, :, s % page, :], want_k[i], dtype, f"k {i}", tol)
        assert torch.equal(vc[s // page, :, (s % page) // vt, :, (s % page) % vt].cpu().float(),
                           qkv[i, hq * D + hkv * D:].reshape(hkv, DV).float()), "v is stored as it is"


def _turn_at(x, rot, p):
    """x [heads, dim] turned as the token at position p is (the plain implementation turns row t by t;
    the two agree on the first rows, which is checked here as well)."""
    R, half = rot["dims"], rot["dims"] // 2
    out = x.clone()
    for i in range(half):
        angle = p * rot["base"] ** (-2.0 * i / R) / rot["scaling"]["factor"]
        c, s = math.cos(angle), math.sin(angle)
        out[:, i] = x[:, i] * c - x[:, i + half] * s
        out[:, i + half] = x[:, i + half] * c + x[:, i] * s
    return out


def test_the_plain_rotation_turns_row_t_by_position_t():
    rot = {"dims": 6, "base": 50.0, "scaling": {"factor": 1.5}}
    x = torch.randn((7, 2, 10), generator=torch.Generator().manual_seed(1), dtype=torch.float64)
    want = torch.stack([_turn_at(x[t], rot, t) for t in range(7)])
    assert float((plain.turn_heads(x, rot) - want).abs().max()) < 1e-12


# ------------------------------------------------------------------------------ chunked attention
def _attention_case(dtype, dev, hq, hkv, D, DV, page, lens, q_lens, seed, chunk, boost=None, free_passed=False):
    """Requests with kv lengths `lens`, the last q_lens of which are this step's queries; keys and values
    over shuffled pages (what unused slots hold must not matter: NaN).  boost = (request, key): that key
    is made the one its request's queries prefer by far.  free_passed: pages wholly before the chunk of a
    request's first query are taken out of its table, as the cache manager gives them back."""
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
        first_needed = ((n - q_lens[s]) // chunk * chunk) // page if free_passed else 0
        tables[s, first_needed: len(mine)] = torch.tensor(mine[first_needed:], dtype=torch.int32)
        kk = torch.randn((n, hkv, D), generator=g).to(dtype)
        vv = torch.randn((n, hkv, DV), generator=g).to(dtype)
        qq = torch.randn((n, hq, D), generator=g).to(dtype)
        if boost is not None and boost[0] == s:
            kk[boost[1]] = 0
            kk[boost[1], :, 0] = 8.0
            qq[:] = 0
            qq[:, :, 0] = 8.0
        for j in range(n):
            if j // page >= first_needed:
                kc[mine[j // page], :, j % page, :] = kk[j].to(dev)
                vc[mine[j // page], :, (j % page) // vt, :, (j % page) % vt] = vv[j].to(dev)
        ks.append(kk), vs.append(vv), qs.append(qq)
        token_seq += [s] * q_lens[s]
        positions += list(range(n - q_lens[s], n))
    q = torch.cat([qs[s][lens[s] - q_lens[s]:] for s in range(S)]).reshape(sum(q_lens), hq * D).contiguous().to(dev)
    assert all(a == 1 or b != 1 for a, b in zip(q_lens, q_lens[1:])), "single tokens come first in a batch"
    batch = SimpleNamespace(
        num_seqs=S, num_tokens=sum(q_lens), token_seq=torch.tensor(token_seq, dtype=torch.int32, device=dev),
        positions=torch.tensor(positions, dtype=torch.int32, device=dev), max_kv_len=max(lens), max_q_len=max(q_lens),
        kv_lens=torch.tensor(lens, dtype=torch.int32, device=dev),
        cu_seqlens_q=torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32, device=dev),
        num_decode=next((i for i, n in enumerate(q_lens) if n != 1), len(q_lens)), q_lens=list(q_lens),
        starts=[n - m for n, m in zip(lens, q_lens)],
        groups=[SimpleNamespace(block_tables=tables.to(dev), slot_mapping=None)])
    return q, kc, vc, batch, (qs, ks, vs)


def _chunk_softmax(qs, ks, vs, lens, q_lens, scale, chunk):
    rows = []
    for q, k, v, n, m in zip(qs, ks, vs, lens, q_lens):
        hq, hkv = q.shape[1], k.shape[1]
        for i in range(n - m, n):
            lo = i // chunk * chunk
            heads = []
            for h in range(hq):
                s = (k[lo: i + 1, h // (hq // hkv)].double() @ q[i, h].double()) * scale
                heads.append(torch.softmax(s, 0) @ v[lo: i + 1, h // (hq // hkv)].double())
            rows.append(torch.cat(heads))
    return torch.stack(rows)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,D,DV,page,chunk,lens,q_lens", [
    (4, 2, 16, 24, 8, 10, [31, 10, 11, 57, 40], [1, 1, 1, 57, 13]),          # decoded tokens at a chunk's last, first and second place
    (6, 2, 24, 40, 16, 33, [200, 67, 150], [1, 67, 85]),                       # portions over several chunks, cut inside one
    (3, 3, 6, 10, 4, 1, [9, 5], [1, 5]),                                       # a chunk of one position: a token reads itself
    (2, 1, 64, 64, 32, 48, [97, 300], [1, 204]),                               # sizes of the matrix-core kind
    (2, 2, 8, 8, 4, 4096, [70, 130], [1, 130]),                                # a chunk longer than every request
    (8, 2, 128, 128, 64, 96, [500, 260], [1, 260])])
def test_chunked_attention_in_prompts_and_decoding(backend, dtype, hq, hkv, D, DV, page, chunk, lens, q_lens):
    k, dev = _kernels(backend, dtype)
    for free_passed in (False, True):
        q, kc, vc, batch, (qs, ks, vs) = _attention_case(dtype, dev, hq, hkv, D, DV, page, lens, q_lens, 5, chunk,
                                                         free_passed=free_passed)
        got = k.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, 0.2, None, v_head_dim=DV, chunk=chunk)
        k.check_faults()
        _close(got, _chunk_softmax(qs, ks, vs, lens, q_lens, 0.2, chunk), dtype, (chunk, free_passed))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,DV", [(16, 24), (64, 64)])
def test_a_key_just_inside_and_just_outside_the_chunk(backend, dtype, D, DV):
    """One key that every query prefers by far, at the chunk's first place, its last, and at the last
    place of the chunk before: seen, seen, not seen; in a prompt's portion and by a decoded token."""
    k, dev = _kernels(backend, dtype)
    chunk, page = 40, 16
    for q_len in (1, 25):
        for n in (chunk * 7 + 1, chunk * 7 + 26, chunk * 8):          # the last query at a chunk's first place, inside, at its last
            if n - q_len < 0:
                continue
            start_of_chunk = (n - 1) // chunk * chunk
            for key, seen in ((start_of_chunk, True), (n - 1, True), (start_of_chunk - 1, False), (3, False)):
                q, kc, vc, batch, (qs, ks, vs) = _attention_case(dtype, dev, 2, 1, D, DV, page, [n], [q_len], 7, chunk,
                                                                 boost=(0, key))
                got = k.paged_attention(q, 2, 1, D, kc, vc, batch, 0, 1.0, None, v_head_dim=DV, chunk=chunk)
                last = got[-1].float().cpu().reshape(2, DV)
                favourite = vs[0][key, 0].float()
                hit = float((last[0] - favourite).abs().max()) < 0.05
                assert hit == seen, (q_len, n, key, seen)
                _close(got, _chunk_softmax(qs, ks, vs, [n], [q_len], 1.0, chunk), dtype, (q_len, n, key))


# ------------------------------------------------------------------------------ state-space layer
def _ssm_weights(heads, vdim, n_state, groups, taps, norm_groups, seed, dtype, slow=None):
    g = torch.Generator().manual_seed(seed)
    inner, gn = heads * vdim, groups * n_state
    C = inner + 2 * gn
    w = {"conv": (torch.randn((C, taps), generator=g) * 0.5).to(dtype), "conv.b": (torch.randn(C, generator=g) * 0.3).to(dtype),
         "dt_bias": torch.randn(heads, generator=g) - 0.5, "A_log": torch.log(0.2 + 3 * torch.rand(heads, generator=g)),
         "D": torch.randn(heads, generator=g), "norm": 1 + 0.4 * torch.randn(inner, generator=g)}
    if slow is not None:
        w["A_log"][slow] = -12.0           # a head that forgets next to nothing
    return w


def _plain_ssm_of_projections(proj, w, heads, vdim, n_state, groups, norm_groups, eps):
    """The plain layer on given projections: an input matrix of one makes them the layer's input."""
    width = proj.shape[1]
    weights = {".in": torch.eye(width, dtype=torch.float64), ".o": torch.eye(heads * vdim, dtype=torch.float64)}
    weights.update({"." + k: v.double() for k, v in w.items()})
    m = {"heads": heads, "vdim": vdim, "state": n_state, "groups": groups, "norm_groups": norm_groups}
    return plain.state_space(proj.double(), m, weights, "", eps)


def _state_batch(dev, q_lens, starts, slots):
    token_seq = [s for s, n in enumerate(q_lens) for _ in range(n)]
    return SimpleNamespace(
        num_seqs=len(q_lens), q_lens=list(q_lens), starts=list(starts),
        num_decode=next((i for i, n in enumerate(q_lens) if n != 1), len(q_lens)),
        token_seq=torch.tensor(token_seq, dtype=torch.int32, device=dev),
        positions=torch.tensor([p for s, n in zip(starts, q_lens) for p in range(s, s + n)], dtype=torch.int32, device=dev),
        cu_seqlens_q=torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32, device=dev),
        seq_starts=torch.tensor(starts, dtype=torch.int32, device=dev),
        state_slots=torch.tensor(slots, dtype=torch.int32, device=dev))


def _run_ssm(k, dev, proj, w, shape, eps, states, q_lens, starts, slots):
    heads, vdim, n_state, groups, taps, norm_groups = shape
    return k.state_space(proj.to(dev), heads, vdim, n_state, groups, taps, w["conv"].to(dev), w["conv.b"].to(dev),
                         w["dt_bias"].to(dev), w["A_log"].to(dev), w["D"].to(dev), w["norm"].to(dev), norm_groups, eps,
                         states[0], states[1], _state_batch(dev, q_lens, starts, slots))


def _new_states(dev, slots, shape, fill=0.0):
    heads, vdim, n_state, groups, taps, _ = shape
    C = heads * vdim + 2 * groups * n_state
    return (torch.full((slots, C, taps - 1), fill, dtype=torch.float32, device=dev),
            torch.full((slots, heads, n_state, vdim), fill, dtype=torch.float32, device=dev))


SSM_SHAPES = [(3, 8, 12, 1, 3, 3), (4, 6, 5, 2, 2, 1), (2, 10, 7, 2, 1, 2), (1, 20, 40, 1, 5, 4), (2, 64, 64, 1, 4, 1),
              (2, 70, 130, 2, 4, 1)]


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", SSM_SHAPES)
def test_state_space_in_portions_of_every_size_and_token_by_token(backend, dtype, shape):
    k, dev = _kernels(backend, dtype)
    heads, vdim, n_state, groups, taps, norm_groups = shape
    T = 75
    g = torch.Generator().manual_seed(4)
    proj = torch.randn((T, 2 * heads * vdim + 2 * groups * n_state + heads), generator=g).to(dtype)
    w = _ssm_weights(heads, vdim, n_state, groups, taps, norm_groups, 9, dtype)
    want = _plain_ssm_of_projections(proj, w, heads, vdim, n_state, groups, norm_groups, 1e-5)
    for portions in ([T], [1] * T, [2] * 3 + [1, 3, 1, 64], [70, 2, 3], [1, 1, 73]):
        states = _new_states(dev, 3, shape, fill=float("nan"))          # what a slot held before must not matter
        out, at = [], 0
        for n in portions:
            out.append(_run_ssm(k, dev, proj[at:at + n], w, shape, 1e-5, states, [n], [at], [1]))
            at += n
        _close(torch.cat(out), want, dtype, portions, tol=4e-2 if dtype == torch.bfloat16 else 1e-4)


@pytest.mark.parametrize("backend", BACKENDS)
def test_state_space_of_unequal_requests_in_one_batch(backend):
    k, dev = _kernels(backend)
    shape = (3, 8, 12, 1, 3, 3)
    heads, vdim, n_state, groups, taps, norm_groups = shape
    width = 2 * heads * vdim + 2 * groups * n_state + heads
    g = torch.Generator().manual_seed(6)
    w = _ssm_weights(*shape, 10, torch.float32)
    lens = [30, 1, 17, 90, 2]
    projs = [torch.randn((n, width), generator=g) for n in lens]
    want = [_plain_ssm_of_projections(p, w, heads, vdim, n_state, groups, norm_groups, 1e-6) for p in projs]
    states = _new_states(dev, 6, shape, fill=float("nan"))
    slots = [4, 0, 2, 5, 1]
    # step 1: every request's first part; steps 2 and 3: single tokens first, portions after them
    cuts = [[29, 1], [1], [10, 1, 6], [3, 80, 7], [1, 1]]
    got = [[] for _ in lens]
    at = [0] * len(lens)
    for step in range(3):
        live = [i for i in range(len(lens)) if step < len(cuts[i])]
        live.sort(key=lambda i: (cuts[i][step] != 1, i))
        rows = torch.cat([projs[i][at[i]:at[i] + cuts[i][step]] for i in live])
        y = _run_ssm(k, dev, rows, w, shape, 1e-6, states, [cuts[i][step] for i in live], [at[i] for i in live],
                     [slots[i] for i in live])
        r = 0
        for i in live:
            got[i].append(y[r:r + cuts[i][step]])
            r += cuts[i][step]
            at[i] += cuts[i][step]
    for i in range(len(lens)):
        _close(torch.cat(got[i]), want[i], torch.float32, i, tol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_state_space_of_long_portions_whose_blocks_run_side_by_side(dtype):
    k, dev = _kernels("hip", dtype)
    shape = (2, 64, 32, 1, 4, 2)
    heads, vdim, n_state, groups, taps, norm_groups = shape
    width = 2 * heads * vdim + 2 * groups * n_state + heads
    g = torch.Generator().manual_seed(8)
    w = _ssm_weights(*shape, 11, dtype, slow=0)
    lens = [1, 700, 65, 64, 129]
    projs = [(torch.randn((n, width), generator=g)).to(dtype) for n in lens]
    want = torch.cat([_plain_ssm_of_projections(p, w, heads, vdim, n_state, groups, norm_groups, 1e-6) for p in projs])
    states = _new_states(dev, 5, shape, fill=float("nan"))
    got = _run_ssm(k, dev, torch.cat(projs), w, shape, 1e-6, states, lens, [0] * 5, [0, 1, 2, 3, 4])
    # (bfloat16 rounds the convolution's output, which the head that forgets nothing sums up over 700 tokens)
    _close(got, want, dtype, "side by side", tol=8e-2 if dtype == torch.bfloat16 else 2e-4)
    kept = [s.clone() for s in states]
    k.state_space_blocks_side_by_side = False
    try:
        states = _new_states(dev, 5, shape, fill=float("nan"))
        one = _run_ssm(k, dev, torch.cat(projs), w, shape, 1e-6, states, lens, [0] * 5, [0, 1, 2, 3, 4])
    finally:
        k.state_space_blocks_side_by_side = True
    _close(got, one.cpu(), dtype, "one after the other", tol=1e-2 if dtype == torch.bfloat16 else 2e-4)
    for a, b in zip(kept, states):
        _close(a, b.cpu(), torch.float32, "the states left behind", tol=2e-4)
    # the blocks from a zero state as products on the matrix cores: the same outputs and states
    k.state_space_shape = 6
    try:
        states = _new_states(dev, 5, shape, fill=float("nan"))
        prod = _run_ssm(k, dev, torch.cat(projs), w, shape, 1e-6, states, lens, [0] * 5, [0, 1, 2, 3, 4])
    finally:
        k.state_space_shape = 0
    _close(got, prod.cpu(), dtype, "as products", tol=1e-2 if dtype == torch.bfloat16 else 2e-4)
    for a, b in zip(kept, states):
        _close(a, b.cpu(), torch.float32, "the states the products left", tol=2e-4)
    # and the next portion goes on from the state the blocks left
    more = (torch.randn((40, width), generator=g)).to(dtype)
    both = _plain_ssm_of_projections(torch.cat((projs[1], more)), w, heads, vdim, n_state, groups, norm_groups, 1e-6)[700:]
    nxt = _run_ssm(k, dev, more, w, shape, 1e-6, kept, [40], [700], [1])
    _close(nxt, both, dtype, "after the blocks", tol=8e-2 if dtype == torch.bfloat16 else 2e-4)


@pytest.mark.parametrize("backend", BACKENDS)
def test_state_space_keeps_a_far_token_by_its_decay(backend):
    """A head that forgets next to nothing carries one early token through hundreds of others, a head
    that forgets fast does not: the early token's mark is in the output 300 tokens on, or gone."""
    k, dev = _kernels(backend)
    shape = (2, 4, 6, 1, 2, 2)
    heads, vdim, n_state, groups, taps, norm_groups = shape
    width = 2 * heads * vdim + 2 * groups * n_state + heads
    g = torch.Generator().manual_seed(12)
    w = _ssm_weights(*shape, 13, torch.float32, slow=0)
    w["A_log"][1] = 1.5
    w["dt_bias"][:] = 0.5
    w["conv"][: heads * vdim, -1] = 1.0                # the mark passes the convolution and its silu
    T = 330
    base = torch.randn((T, width), generator=g) * 0.3
    marked = base.clone()
    marked[5, heads * vdim: 2 * heads * vdim] += 25.0          # a large x at token 5
    outs = []
    for proj in (base, marked):
        states = _new_states(dev, 1, shape)
        y = torch.cat([_run_ssm(k, dev, proj[a:b], w, shape, 1e-6, states, [b - a], [a], [0])
                       for a, b in ((0, 100), (100, 101), (101, 329), (329, 330))])
        want = _plain_ssm_of_projections(proj, w, heads, vdim, n_state, groups, norm_groups, 1e-6)
        _close(y, want, torch.float32, "plain", tol=1e-4)
        outs.append(y.cpu())
    moved = (outs[1][-1] - outs[0][-1]).abs().reshape(heads, vdim).max(-1).values
    assert float(moved[0]) > 1e-2 and float(moved[1]) < 1e-5, moved


# ------------------------------------------------------------------------------ routed feed-forward
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,top,count,keep", [(6, 2, 3, 2), (4, 1, 1, 1), (5, 3, 5, 3), (9, 2, 3, 1), (14, 2, 2, 1), (64, 6, 8, 3)])
def test_the_choice_of_experts(backend, experts, top, count, keep):
    k, dev = _kernels(backend)
    g = torch.Generator().manual_seed(experts)
    logits = torch.randn((40, experts), generator=g) * 2
    # a token whose best expert sits in a poor group: the group rule keeps it out
    if count > keep and experts // count > 1:
        per = experts // count
        logits[0] = -3.0 - 0.01 * torch.arange(experts)
        logits[0, 0] = 5.0                              # group 0: one very good expert, the others poor
        logits[0, per: 2 * per] = 2.0 + 0.01 * torch.arange(per)      # group 1: all good
    ids, weights = k.moe_route(logits.to(dev), top, count, keep, 1.7)
    router = {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}
    for t in range(logits.shape[0]):
        s = torch.sigmoid(logits[t].double())
        want = plain.choose_experts(s, router)
        assert sorted(ids[t].tolist()) == sorted(want), t
        for e, wt in zip(ids[t].tolist(), weights[t].tolist()):
            assert abs(wt - 1.7 * float(s[e])) < 1e-5
    if count > keep and experts // count > 1 and keep == 1:
        assert 0 not in ids[0].tolist()


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,width,ff,experts,top", [(1, 48, 20, 6, 2), (7, 20, 9, 5, 3), (150, 72, 30, 10, 2), (33, 128, 64, 8, 3),
                                                         (40, 72, 40, 6, 2), (300, 64, 32, 4, 2), (700, 160, 104, 5, 2), (8, 256, 128, 32, 6)])
def test_the_experts_products(backend, dtype, tokens, width, ff, experts, top):
    k, dev = _kernels(backend, dtype)
    g = torch.Generator().manual_seed(tokens)
    x = torch.randn((tokens, width), generator=g).to(dtype)
    up = (torch.randn((experts * ff, width), generator=g) * 0.3).to(dtype)
    down = (torch.randn((experts * width, ff), generator=g) * 0.3).to(dtype)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(tokens)]).to(torch.int32)
    if tokens > 100:
        ids[:90, 0] = experts - 1                        # two experts with more rows than a tile holds
        ids[:90, 1] = experts - 2
        ids[:90, 2:] = torch.arange(top - 2)[None, :]
    weights = torch.rand((tokens, top), generator=g) + 0.2
    add = torch.randn((tokens, width), generator=g).to(dtype)
    w = {}
    for e in range(experts):
        w[f".e{e}.up"] = up[e * ff:(e + 1) * ff].double()
        w[f".e{e}.down"] = down[e * width:(e + 1) * width].double()
    want = add.double().clone()
    for t in range(tokens):
        for c in range(top):
            want[t] += float(weights[t, c]) * plain.expert(x[t].double(), w, f".e{int(ids[t, c])}")
    got = k.moe_experts(x.to(dev), ids.to(dev), weights.to(dev), up.to(dev), down.to(dev), experts, "relu2", add=add.to(dev))
    _close(got, want, dtype, "experts", tol=3e-2 if dtype == torch.bfloat16 else 1e-4)
    none = k.moe_experts(x.to(dev), ids.to(dev), weights.to(dev), up.to(dev), down.to(dev), experts, "relu2")
    _close(none, want - add.double(), dtype, "without the addend", tol=3e-2 if dtype == torch.bfloat16 else 1e-4)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_activations_without_a_gate(backend, dtype):
    k, dev = _kernels(backend, dtype)
    x = (torch.randn((5, 33), generator=torch.Generator().manual_seed(1)) * 3).to(dtype)
    xd = x.double()
    for act, want in (("relu2", torch.relu(xd) ** 2), ("relu", torch.relu(xd)), ("silu", xd * torch.sigmoid(xd)),
                      ("gelu_tanh", 0.5 * xd * (1 + torch.tanh(math.sqrt(2 / math.pi) * (xd + 0.044715 * xd ** 3))))):
        _close(k.act(x.to(dev), act), want, dtype, act)
    logits = torch.randn((3, 50))
    _close(k.scale_(logits.clone().to(dev), 2.5), logits.double() * 2.5, torch.float32, "scale")


# ------------------------------------------------------------------------------ the model through the step function
def _runner(name, backend, dtype, pages, max_requests=4):
    kernels, dev = _kernels(backend, torch.float32 if dtype == "float32" else torch.bfloat16)
    return H.make_runner(M.model_folder(name, dtype), dtype, M.CONFIGS[name]["page"], pages, device=dev,
                         kernels=kernels, max_requests=max_requests)


MODEL_TOL = {"float32": 1e-4, "bfloat16": 6e-2}


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_every_cutting_gives_the_plain_logits(backend, name):
    c = M.CONFIGS[name]
    n = 110
    toks = H.random_tokens(c["cfg"].vocab, n, 1)
    want = M.plain_logits(M.model_folder(name), toks)
    r = _runner(name, backend, "float32", 40)
    assert len(r.cache.groups) == len({l.left.chunk for l in c["cfg"].layers}) and r.cache.slots.num_slots == 4
    for portions in (H.whole(n), H.last_one_by_one(n, 45), H.changing_portions(n, 2), [1] * 3 + [2] * 10 + [n - 23]):
        got = H.run_portions(r, "x", toks, portions)
        assert M.err(got, want) < MODEL_TOL["float32"], portions
    assert all(pool.num_free == 40 for pool in r.cache.pools)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["a", "b", "d"])
def test_bfloat16_follows_the_plain_logits_under_every_cutting(name):
    c = M.CONFIGS[name]
    n = 130
    toks = H.random_tokens(c["cfg"].vocab, n, 3)
    want = M.plain_logits(M.model_folder(name, "bfloat16"), toks)
    r = _runner(name, "hip", "bfloat16", 40)
    for portions in (H.whole(n), H.last_one_by_one(n, 40), H.changing_portions(n, 4)):
        e = M.errors(H.run_portions(r, "x", toks, portions), want)
        # rounding may give a token another expert where two scores lie close: few positions, none far off
        assert float(e.median()) < MODEL_TOL["bfloat16"] / 2 and float((e > MODEL_TOL["bfloat16"]).float().mean()) <= 0.05 \
            and float(e.max()) < 0.6, (portions, float(e.median()), float(e.max()))


@pytest.mark.gpu
def test_a_larger_model_over_long_prompts():
    """Six hundred tokens through a model of three cache groups: whole (the recurrence in blocks side by side, keys
    hundreds of positions back inside the longest chunk), in changing portions, and its last tokens one by one."""
    name = "e"
    c = M.CONFIGS[name]
    n = 600
    toks = H.random_tokens(c["cfg"].vocab, n, 17)
    want = M.plain_logits(M.model_folder(name), toks)
    r = _runner(name, "hip", "float32", 12)
    assert len(r.cache.groups) == 3
    for portions in (H.whole(n), H.changing_portions(n, 5), H.last_one_by_one(n, 70)):
        assert M.err(H.run_portions(r, "x", toks, portions), want) < MODEL_TOL["float32"], portions[:4]
    assert all(pool.num_free == 12 for pool in r.cache.pools)


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_first_tokens_of_a_sequence(backend):
    for name in ("a", "c"):
        c = M.CONFIGS[name]
        r = _runner(name, backend, "float32", 8)
        for n in (1, 2, 3, 5):
            toks = H.random_tokens(c["cfg"].vocab, n, 40 + n)
            want = M.plain_logits(M.model_folder(name), toks)
            for portions in ([n], [1] * n):
                assert M.err(H.run_portions(r, "x", toks, portions), want) < MODEL_TOL["float32"], (name, n, portions)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["a", "c"])
def test_long_decoding(backend, name):
    # one prompt token, then 170 tokens one by one: over pages and chunks, the state carried all the way
    c = M.CONFIGS[name]
    n = 171
    toks = H.random_tokens(c["cfg"].vocab, n, 5)
    want = M.plain_logits(M.model_folder(name), toks)
    r = _runner(name, backend, "float32", 48)
    assert M.err(H.run_portions(r, "x", toks, [1] * n), want) < MODEL_TOL["float32"]
    if name == "a":
        # a chunked group holds the pages of the chunk at hand only: the others went back on the way
        r.cache.admit("y")
        for pos in range(n):
            r.cache.reserve("y", pos + 1)
        held = [sum(1 for p in t if p >= 0) for t in r.cache.requests["y"].tables]
        assert max(held) <= 3 and len(r.cache.requests["y"].tables[0]) == (n + 7) // 8, held
        r.cache.release("y")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["a", "d"])
def test_mixed_batches_on_pages_and_slots_that_are_used_again(backend, name):
    c = M.CONFIGS[name]
    lens = {"r0": 60, "r1": 41, "r2": 77, "r3": 1, "r4": 35, "r5": 52, "r6": 66, "r7": 2}
    reqs = {r: H.random_tokens(c["cfg"].vocab, n, i) for i, (r, n) in enumerate(lens.items())}
    pages = 192 // c["page"]                   # 192 tokens of cache and three state slots for 334 tokens of eight requests
    r = _runner(name, backend, "float32", pages, max_requests=3)
    got = H.run_mixed(r, reqs, seed=3, max_live=3)
    for rid, toks in reqs.items():
        assert M.err(got[rid], M.plain_logits(M.model_folder(name), toks)) < MODEL_TOL["float32"], rid
    assert all(pool.num_free == pages for pool in r.cache.pools) and r.cache.slots.num_free == 3
    # each request alone gives what it gave in the batches
    alone = _runner(name, backend, "float32", pages, max_requests=1)
    for rid in ("r1", "r3", "r6"):
        one = H.run_portions(alone, rid, reqs[rid], [len(reqs[rid])])
        assert M.err(got[rid], one) < 1e-5, rid


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_residual_stream_after_every_layer(backend):
    """Layer by layer: the float32 stream after a layer is the plain implementation's."""
    name = "a"
    c = M.CONFIGS[name]
    toks = H.random_tokens(c["cfg"].vocab, 37, 9)
    cfg, w = M.plain_model(M.model_folder(name))
    _, streams = plain.forward(cfg, w, toks, return_layers=True)
    r = _runner(name, backend, "float32", 8)
    seen = []
    inner = r.kernels.stream_dyt

    def spy(addends, residual, *a, **kw):
        y, res = inner(addends, residual, *a, **kw)
        seen.append(res.detach().float().cpu().clone())
        return y, res
    r.kernels.stream_dyt = spy
    try:
        H.run_portions(r, "x", toks, [len(toks)])
    finally:
        del r.kernels.stream_dyt
    # the stream is seen by every norm: two a layer with a feed-forward, one without, and the final one
    at, ends = 0, []
    for layer in cfg["layers"]:
        at += 2 if layer.get("mlp") else 1
        ends.append(at)                                   # the norm that first sees the stream after this layer
    assert len(seen) == at + 1
    for i, want in enumerate(streams):
        assert float((seen[ends[i]].double() - want).abs().max() / want.abs().max()) < 2e-5, i


# ------------------------------------------------------------------------------ the engine
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("schedule", ["prefill_first", "mixed"])
def test_greedy_generation_through_the_engine(backend, schedule):
    name = "d"
    c = M.CONFIGS[name]
    kernels, dev = _kernels(backend)
    folder = M.model_folder(name)
    prompts = [H.random_tokens(c["cfg"].vocab, n, 60 + n) for n in (3, 30, 1, 47, 18)]
    # few pages, three request slots and portions of at most 16 tokens: prompts are cut, requests wait
    llm = LLM(folder, kernels=kernels, device=dev, dtype="float32", kvcache_block_size=c["page"], num_kvcache_blocks=10,
              max_num_batched_tokens=16, max_num_seqs=3, schedule=schedule, max_model_len=128)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True), use_tqdm=False)
    cfg, w = M.plain_model(folder)
    for p, o in zip(prompts, outs):
        assert o["token_ids"] == plain.greedy_generate(cfg, w, p, 10), len(p)
    assert llm.runner.cache.slots.num_free == 3 and all(pool.num_free == 10 for pool in llm.runner.cache.pools)


@pytest.mark.gpu
def test_generation_in_bfloat16_with_captured_steps_and_bursts():
    name = "b"
    c = M.CONFIGS[name]
    folder = M.model_folder(name, "bfloat16")
    prompts = [H.random_tokens(c["cfg"].vocab, n, 80 + n) for n in (5, 40, 90, 17)]
    sp = SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True)
    common = dict(dtype="bfloat16", kvcache_block_size=c["page"], num_kvcache_blocks=24, max_num_seqs=4, max_model_len=256)
    eager = LLM(folder, enforce_eager=True, **common).generate(prompts, sp, use_tqdm=False)
    graphs = LLM(folder, decode_burst=8, **common)
    assert graphs.runner._graph_max_batch, "the state-space layer reads the step's metadata on the device: its steps are captured"
    fast = graphs.generate(prompts, sp, use_tqdm=False)
    for a, b in zip(eager, fast):
        assert a["token_ids"] == b["token_ids"]


@pytest.mark.gpu
def test_trace_replay_of_a_model_folder(tmp_path):
    """bin/trace_run as a process on a Mafarax folder: portions, single tokens and a second request that
    takes the first one's pages and slot."""
    import os
    import subprocess
    import sys
    import numpy as np
    name = "d"
    c = M.CONFIGS[name]
    folder = M.model_folder(name)
    a, b = H.random_tokens(c["cfg"].vocab, 50, 1), H.random_tokens(c["cfg"].vocab, 70, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:33], "want": [0, 32]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[33:34], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[34:], "want": [15]}, {"id": "b", "tokens": b[:2], "want": []}], "end": ["a"]},
             {"step": 3, "entries": [{"id": "b", "tokens": b[2:], "want": [67]}], "end": ["b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                           "--out", str(out), "--max-tokens", "128", "--page-size", str(c["page"])],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", text=True, capture_output=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    wa, wb = M.plain_logits(folder, a), M.plain_logits(folder, b)
    V = c["cfg"].vocab
    read = lambda i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V))
    assert M.err(read(0), wa[[0, 32]]) < 1e-4 and M.err(read(1), wa[[33]]) < 1e-4
    assert M.err(read(2), wa[[49]]) < 1e-4 and M.err(read(3), wb[[69]]) < 1e-4
