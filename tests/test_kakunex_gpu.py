"""Kakunex on the GPU against the plain implementation (``tests/plain/kakunex_plain.py``): every mechanism alone on
inputs made so that a fault shows, then whole models with random weights under every kind of schedule: whole
prompts, token-by-token decoding, portions down to two tokens, batches of unequal requests, pages and state slots
that are given back and used again, long decoding, greedy generation through the engine and its scheduler, and the
trace replay tool."""

from __future__ import annotations

import copy
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from kakunex_models import KAKUNEX, make_folder
from plain import kakunex_plain as K
from plain.model_folder import read_model_folder
from tolerances import check_logits

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def ops():
    from miniserve_amd.kernels import ops as o

    o.library()
    return o


def dev(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV).contiguous()


def close(got, want, dtype, what=""):
    got = got.float().cpu().numpy().astype(np.float64)
    scale = max(float(np.abs(want).max()), 1e-30)
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    worst = float(np.abs(got - want).max())
    assert worst <= tol * scale, f"{what}: max |diff| {worst:.3e} > {tol * scale:.3e}"


# ---------------------------------------------------------------- mechanisms alone


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [1, 7, 64, 200, 1030])
def test_layer_norm(width, out_dtype):
    rng = np.random.default_rng(width)
    x = rng.normal(size=(9, width)) * 3 + 5  # a mean far from zero: a variance taken as E[x^2] - mean^2 would lose digits
    w, b = rng.normal(size=width), rng.normal(size=width)
    want = K.layer_norm(x, w, b, 1e-5)
    got = ops().layernorm(dev(x), dev(w), dev(b), 1e-5, out_dtype)
    close(got, want, out_dtype, "all rows")
    rows = [8, 0, 3, 3]
    got = ops().layernorm(dev(x), dev(w), dev(b), 1e-5, out_dtype, dev(rows, torch.int32))
    close(got, want[rows], out_dtype, "row list")
    got = ops().layernorm(dev(x), dev(w), None, 1e-5, out_dtype)
    close(got, K.layer_norm(x, w, 0.0, 1e-5), out_dtype, "no bias")


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("groups,group", [(1, 160), (4, 40), (5, 32), (3, 5), (1, 700), (2, 300)])
def test_gated_group_norm(groups, group, out_dtype):
    rng = np.random.default_rng(groups * 1000 + group)
    n = groups * group
    x, w = rng.normal(size=(5, n)) * 4, rng.normal(size=n)
    wide = rng.normal(size=(5, n + 13)) * 2  # the gate is a column slice of a wider matrix
    want = (K.unit_rms(x.reshape(5, groups, group), 1e-6).reshape(5, n)) * w * K.sigmoid(wide[:, 6 : 6 + n])
    got = ops().group_rmsnorm_gate(dev(x), group, dev(w), dev(wide)[:, 6 : 6 + n], 1e-6, out_dtype)
    close(got, want, out_dtype)
    got = ops().group_rmsnorm_gate(dev(x), group, None, None, 1e-6, out_dtype)
    close(got, K.unit_rms(x.reshape(5, groups, group), 1e-6).reshape(5, n), out_dtype, "bare")


@pytest.mark.parametrize("width", [5, 176, 600])
def test_mean_of_normed_streams(width):
    rng = np.random.default_rng(width)
    r, a, b = rng.normal(size=(6, width)), rng.normal(size=(6, width)) * 10, rng.normal(size=(6, width)) * 0.01
    wa, wb = rng.normal(size=width), rng.normal(size=width)
    res = dev(r)
    ops().normed_mean_add(res, [dev(a), dev(b)], [dev(wa), dev(wb)], 1e-6, 0.5)
    close(res, r + 0.5 * (K.rms_norm(a, wa, 1e-6) + K.rms_norm(b, wb, 1e-6)), torch.float32)


@pytest.mark.parametrize("block", [0, 16])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_clamped_gated_activation(block, dtype):
    rng = np.random.default_rng(3)
    inter, lim = 48, 1.5
    g, u = rng.normal(size=(7, inter)) * 3, rng.normal(size=(7, inter)) * 3  # many values beyond the limit, on both sides
    gu = np.concatenate((g, u), axis=1)
    if block:
        gu = np.stack((g.reshape(7, -1, block), u.reshape(7, -1, block)), axis=2).reshape(7, 2 * inter)
    gc = np.minimum(g, lim)
    want = gc * K.sigmoid(1.702 * gc) * (np.clip(u, -lim, lim) + 1)
    if dtype == torch.bfloat16:
        gq = dev(gu, dtype).float().cpu().numpy().astype(np.float64)  # what the kernel is given
        g2, u2 = (gq[:, :inter], gq[:, inter:]) if not block else (gq.reshape(7, -1, 2, block)[:, :, 0].reshape(7, inter),
                                                                    gq.reshape(7, -1, 2, block)[:, :, 1].reshape(7, inter))
        gc = np.minimum(g2, lim)
        want = gc * K.sigmoid(1.702 * gc) * (np.clip(u2, -lim, lim) + 1)
    got = ops().act_mul(dev(gu, dtype), "swiglu_clamped", block=block, limit=lim)
    close(got, want, dtype)
    parts = dev(np.stack((gu * 0.25, gu * 0.75)))
    got = ops().act_mul(ops().SplitSum(parts), "swiglu_clamped", out_dtype=torch.float32, block=block, limit=lim)
    if dtype == torch.float32:
        close(got, want, dtype, "partial sums")
    with pytest.raises(ValueError):
        ops().act_mul(dev(gu, dtype), "swiglu_clamped", block=block)


def step_batch(lens, starts, slots=None):
    """What the kernels read of a step: rows of ``lens`` new tokens behind ``starts`` cached ones."""
    pos = np.concatenate([np.arange(s, s + n) for n, s in zip(lens, starts)])
    row = np.concatenate([np.full(n, i) for i, n in enumerate(lens)])
    b = SimpleNamespace(num_rows=len(lens), num_tokens=int(sum(lens)), positions=dev(pos, torch.int32), token_row=dev(row, torch.int32),
                        row_start=dev(np.concatenate(([0], np.cumsum(lens))), torch.int32), starts=dev(starts, torch.int32),
                        state_slots=dev(slots if slots is not None else list(range(len(lens))), torch.int32),
                        num_decode_tokens=sum(1 for n in lens if n == 1), decode_tokens=None, prefill_tokens=None,
                        max_kv_len=max(s + n for n, s in zip(lens, starts)), row_lens=list(lens), row_starts_host=list(starts), memo={})
    b.is_decode = b.num_decode_tokens == len(lens)
    return b


def plain_attention(q, k, v, scale, size, keep, groups):
    """``q [T, H, D]``, ``k [T, G, D]``, ``v [T, G, E]`` of one sequence; float64."""
    T, H, _ = q.shape
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        js = [j for j in range(i + 1) if K.visible(i, j, size or T + 1, keep)]
        for a in range(H):
            s = (k[js, a // groups] @ q[i, a]) * scale
            p = np.exp(s - s.max())
            out[i, a] = (p / p.sum()) @ v[js, a // groups]
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,E,rot,pairing,size,keep", [
    (4, 2, 16, 24, 8, "adjacent", 12, 5),    # keys and values of different sizes, part of the head turned
    (3, 3, 20, 12, 20, "adjacent", 16, 17),  # a head size that is no multiple of 8; more kept keys than a page
    (6, 1, 64, 64, 0, "halves", 33, 0),      # no rotation, a window without kept keys, one key/value head
    (2, 2, 8, 40, 6, "halves", 0, 0),        # every key visible
    (2, 1, 32, 32, 16, "adjacent", 45, 19),
    (2, 1, 128, 128, 32, "adjacent", 70, 9),   # the largest head the tiled kernel takes
    (2, 1, 96, 16, 32, "adjacent", 30, 7),     # the matrix-core form's other sizes: keys of 96, values of 16
    (1, 1, 160, 136, 0, "halves", 50, 3),      # beyond it: the kernel with a wave (or several) per token and head
])
def test_window_attention_with_kept_first_keys(H, G, D, E, rot, pairing, size, keep, dtype):
    """Norm over the whole projection, rotation, cache store and attention against the plain formulas, in one step and
    cut into portions and single tokens. A few tokens' keys are long, every query looks along them and their values are large, so that the
    softmax is decided by which of those keys is visible: a window, or a run of kept keys, that is one token off moves
    the output by its own size."""
    o = ops()
    rng = np.random.default_rng(H * 100 + D)
    T, page = 150, 16
    qkv = rng.normal(size=(T, H * D + G * D + G * E))
    mark = rng.normal(size=D)
    stride = max(7, size // 2 + 1)  # one or two marked keys in a window
    marked = sorted(set(range(0, T, stride)) | ({keep - 1} if keep else set()))
    for g in range(G):
        qkv[marked, H * D + g * D : H * D + (g + 1) * D] = 3 * mark + 0.1 * rng.normal(size=(len(marked), D))
    qkv[marked, H * D + G * D :] *= 4  # and their values are large
    for a in range(H):
        qkv[:, a * D : (a + 1) * D] += 2 * mark
    qw, kw = rng.uniform(0.5, 1.5, size=H * D), rng.uniform(0.5, 1.5, size=G * D)
    eps, scale = 1e-6, 0.8
    q = K.rms_norm(qkv[:, : H * D], qw, eps).reshape(T, H, D)
    k = K.rms_norm(qkv[:, H * D : H * D + G * D], kw, eps).reshape(T, G, D)
    v = qkv[:, H * D + G * D :].reshape(T, G, E)
    freqs = 30.0 ** (-np.arange(rot // 2) * 2.0 / max(rot, 1))
    if rot:
        if pairing == "adjacent":
            q, k = K.rotate_adjacent(q, np.arange(T), freqs), K.rotate_adjacent(k, np.arange(T), freqs)
        else:
            def halves(x):
                ang = np.arange(T)[:, None] * freqs[None, :]
                c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
                y = x.copy()
                y[..., : rot // 2] = x[..., : rot // 2] * c - x[..., rot // 2 : rot] * s
                y[..., rot // 2 : rot] = x[..., rot // 2 : rot] * c + x[..., : rot // 2] * s
                return y
            q, k = halves(q), halves(k)
    want = plain_attention(q, k, v, scale, size, keep, H // G).reshape(T, H * E)
    # the test's inputs do what they are for: one key more or fewer in the window or among the kept keys shows
    if size:
        off = plain_attention(q, k, v, scale, size + 1, keep, H // G).reshape(T, H * E)
        assert np.abs(off - want).max() > 0.1 * np.abs(want).max()
    if keep:
        off = plain_attention(q, k, v, scale, size, keep - 1, H // G).reshape(T, H * E)
        assert np.abs(off - want).max() > 0.1 * np.abs(want).max()

    pages = -(-T // page)
    for cuts in ([T], [100] + [1] * 50, [2, 3, 64, 5, 2, 31, 1, 1, 40, 1]):
        kc = torch.zeros((pages + 1, G, page, D), dtype=dtype, device=DEV)
        vc = torch.zeros((pages + 1, G, E, page), dtype=dtype, device=DEV)
        table = dev(np.arange(pages)[None, :], torch.int32)  # scattered pages are the model tests' matter
        got, at = [], 0
        for n in cuts:
            n = min(n, T - at)
            if n <= 0:
                break
            b = step_batch([n], [at])
            rope = o.rope_table(b.positions, dev(freqs)) if rot else None
            slots = dev(np.arange(at, at + n), torch.int32)
            qq = o.qkv_norm_rope_store(dev(qkv[at : at + n]), slots, dev(qw), dev(kw), eps, rope, kc, vc, H, G, D, E, dtype, pairing)
            got.append(o.paged_attention(qq, kc, vc, table, b, H, G, D, scale, size, E, keep, True))
            at += n
        got = torch.cat(got)
        if dtype == torch.float32:  # scores are sums of D float32 products and stand in an exponent: the bound grows with D
            err = np.abs(got.cpu().numpy() - want).max()
            assert err <= 2e-5 * max(1.0, D / 64) * np.abs(want).max(), f"cuts {cuts[:3]}: {err:.3e}"
        else:
            err = np.abs(got.float().cpu().numpy() - want)
            assert err.max() <= 0.06 * np.abs(want).max() and np.sqrt((err**2).mean()) <= 0.01 * np.abs(want).max(), f"cuts {cuts[:3]}"


def plain_recurrence(q, k, v, a, b):
    """``S_t = a_t S + b_t k_t v_t^T``, ``o_t = S_t^T q_t`` for one head: ``q, k [T, D]``, ``v [T, E]``, ``a, b [T]``."""
    S = np.zeros((q.shape[1], v.shape[1]))
    out = np.zeros_like(v)
    for t in range(len(q)):
        S = a[t] * S + b[t] * np.outer(k[t], v[t])
        out[t] = S.T @ q[t]
    return out, S


@pytest.mark.parametrize("H,D,E", [(6, 24, 40), (3, 8, 16), (1, 48, 20), (2, 128, 128), (5, 12, 200), (2, 200, 8), (2, 7, 10), (3, 33, 1)])
def test_decay_recurrence_far_keys_and_cuts(H, D, E):
    """One token far back carries a large key and value; a head that hardly decays must still answer a late query along
    that key with it, a head that decays fast must have lost it. Rows of a batch start from their own slots, a row
    that begins its sequence from zero whatever the slot held."""
    o = ops()
    rng = np.random.default_rng(D)
    T = 400
    decay = np.linspace(0.5, 0.9995, H) if H > 1 else np.array([0.999])
    cols = {"q": 3, "k": 3 + H * D, "v": 3 + 2 * H * D}
    x = rng.normal(size=(T, 3 + 2 * H * D + H * E + 2)) * 0.3
    key = rng.normal(size=D)
    for h in range(H):
        x[5, cols["k"] + h * D : cols["k"] + (h + 1) * D] = 4 * key
        x[5, cols["v"] + h * E : cols["v"] + (h + 1) * E] = 6.0
        x[T - 10 :, cols["q"] + h * D : cols["q"] + (h + 1) * D] = 2 * key
    want = np.zeros((T, H * E))
    for h in range(H):
        q, k = (K.silu(x[:, cols[n] + h * D : cols[n] + (h + 1) * D]) for n in ("q", "k"))
        v = K.silu(x[:, cols["v"] + h * E : cols["v"] + (h + 1) * E])
        want[:, h * E : (h + 1) * E], _ = plain_recurrence(q, k, v, np.full(T, decay[h]), np.ones(T))
    last, first = want[-1, (H - 1) * E : H * E], want[-1, :E]
    assert H == 1 or np.abs(last).mean() > 5 * np.abs(first).mean()  # the far token is what the slow head answers with
    state = {"S": torch.full((4, H, D, E), 7.0, device=DEV)}  # what an earlier request left in the slots
    for cuts in ([T], [300] + [1] * 100, [2, 3, 64, 5, 2, 131, 1, 1, 190, 1]):
        got, at = [], 0
        for n in cuts:
            n = min(n, T - at)
            if n <= 0:
                break
            b = step_batch([n], [at], [2])
            got.append(o.gated_recurrence(dev(x[at : at + n]), cols, H, D, E, b, state, mode="decay", activation="silu", decay=dev(decay)))
            at += n
        close(torch.cat(got), want, torch.float32, f"cuts {cuts[:3]}")
    # three rows in one step, each from its own slot: the first 50 tokens of the sequence in slot 0 and in slot 3,
    # and the rest of the sequence above from slot 2
    rest = T - at if at < T else 0
    assert rest == 0
    b = step_batch([50, 1, 50], [0, 0, 0], [0, 1, 3])
    xs = np.concatenate((x[:50], x[:1], x[:50]))
    got = o.gated_recurrence(dev(xs), cols, H, D, E, b, state, mode="decay", activation="silu", decay=dev(decay))
    close(got[:50], want[:50], torch.float32, "row 0")
    close(got[50:51], want[:1], torch.float32, "row 1")
    close(got[51:], want[:50], torch.float32, "row 2")
    b = step_batch([30, 1], [50, 1], [3, 1])
    got = o.gated_recurrence(dev(np.concatenate((x[50:80], x[1:2]))), cols, H, D, E, b, state, mode="decay", activation="silu", decay=dev(decay))
    close(got[:30], want[50:80], torch.float32, "row 0 goes on")
    close(got[30:], want[1:2], torch.float32, "row 1 goes on")


@pytest.mark.parametrize("H,D,E,cap", [(4, 40, 56, 12.0), (2, 8, 24, 3.0), (1, 128, 64, 30.0), (3, 20, 130, 1.0), (2, 6, 9, 4.0), (2, 1, 127, 6.0)])
def test_exponential_gate_recurrence(H, D, E, cap):
    """Gates from far below to far above zero (the cap bounds them), so that the running maximum moves both ways, the
    normaliser's two branches are both taken and a state that started at zero still counts in the maximum. The
    running maximum is a float32 sum of gates as large as the cap: what each addition rounds away (the cap times
    2^-24) stays in the state's scale and shows where the normaliser's floor exp(-m) decides, so the bound grows
    with the cap. And the normaliser n . q is a sum of terms of both signs: where it is small beside them, float32
    has lost what the sum cancelled, in any order of summation, so a token's bound also grows with that ratio."""
    o = ops()
    rng = np.random.default_rng(E)
    T = 300
    cols = {"q": 0, "k": H * D, "v": 2 * H * D, "i": 2 * H * D + H * E + 1, "f": 2 * H * D + H * E + 1 + H}
    x = rng.normal(size=(T, cols["f"] + H)) * 0.5
    x[:, cols["i"] : cols["i"] + H] = rng.normal(size=(T, H)) * 2 * cap
    x[:, cols["f"] : cols["f"] + H] = rng.normal(size=(T, H)) * 3 + 2
    x[:40, cols["i"] : cols["i"] + H] = -abs(x[:40, cols["i"] : cols["i"] + H])  # early on the maximum is the zero state's
    bi, bf = rng.normal(size=H), rng.normal(size=H)
    want = np.zeros((T, H * E))
    lost = np.zeros((T, H * E))  # sum |n_d q_d| over the normaliser, per output element
    branches = set()
    for h in range(H):
        q = x[:, h * D : (h + 1) * D] * D**-0.5
        k = x[:, cols["k"] + h * D : cols["k"] + (h + 1) * D]
        v = x[:, cols["v"] + h * E : cols["v"] + (h + 1) * E]
        gi = cap * np.tanh((x[:, cols["i"] + h] + bi[h]) / cap)
        gf = K.log_sigmoid(cap * np.tanh((x[:, cols["f"] + h] + bf[h]) / cap))
        S, n, m = np.zeros((D, E)), np.zeros(D), 0.0
        for t in range(T):
            m_new = max(gf[t] + m, gi[t])
            S = math.exp(gf[t] + m - m_new) * S + math.exp(gi[t] - m_new) * np.outer(k[t], v[t])
            n = math.exp(gf[t] + m - m_new) * n + math.exp(gi[t] - m_new) * k[t]
            m = m_new
            branches.add(abs(n @ q[t]) > math.exp(-m))
            want[t, h * E : (h + 1) * E] = S.T @ q[t] / (max(abs(n @ q[t]), math.exp(-m)) + 1e-6)
            lost[t, h * E : (h + 1) * E] = np.abs(n * q[t]).sum() / (max(abs(n @ q[t]), math.exp(-m)) + 1e-6)
    assert branches == {True, False}
    state = {"S": torch.full((3, H, D, E), 3.0, device=DEV), "n": torch.full((3, H, D), -2.0, device=DEV),
             "m": torch.full((3, H), 9.0, device=DEV)}
    for cuts in ([T], [200] + [1] * 100, [2, 3, 64, 5, 2, 31, 1, 1, 190, 1]):
        got, at = [], 0
        for n in cuts:
            n = min(n, T - at)
            if n <= 0:
                break
            b = step_batch([n], [at], [1])
            got.append(o.gated_recurrence(dev(x[at : at + n]), cols, H, D, E, b, state, mode="exp_gates", q_scale=D**-0.5, cap=cap,
                                          i_bias=dev(bi), f_bias=dev(bf)))
            at += n
        err = np.abs(torch.cat(got).cpu().numpy() - want)
        bound = 1e-5 * max(2.0, cap) * np.abs(want).max() + 5e-7 * lost * np.abs(want)
        assert (err <= bound).all(), f"cuts {cuts[:3]}: {(err / bound).max():.2f} times the bound"


# ---------------------------------------------------------------- whole models


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("kakunex")
    return {name: make_folder(root, name) for name in KAKUNEX}


@pytest.fixture(scope="module")
def plain_logits(folders):
    memo = {}

    def get(name, tokens):
        key = (name, tuple(tokens))
        if key not in memo:
            cfg, w = read_model_folder(folders[name])
            memo[key] = K.forward(cfg, w, tokens)
        return memo[key]

    return get


def tokens_for(name, n, seed):
    return np.random.default_rng(seed).integers(0, KAKUNEX[name][0]["vocab"], size=n).tolist()


def make_runner(folder, dtype, pool_tokens, slots, **kw):
    from miniserve_amd.engine.runner import ModelRunner
    from miniserve_amd.loading import load_model

    return ModelRunner(load_model(folder, dtype, DEV), kv_pool_tokens=pool_tokens, max_running=slots, **kw)


def run_schedule(runner, requests, steps):
    """``steps``: lists of ``(request, count)``; every position's logits are asked for. A request is admitted at its
    first entry and released when its last token has run. Returns request -> ``[T, vocab]``."""
    from miniserve_amd.engine.batch import StepRow

    at = {r: 0 for r in requests}
    live, got = {}, {r: [] for r in requests}
    for step in steps:
        rows, who = [], []
        for r, n in step:
            if r not in live:
                live[r] = runner.acquire()
            rows.append(StepRow(live[r], requests[r][at[r] : at[r] + n], list(range(n))))
            who += [r] * n
            at[r] += n
        logits = runner.step(rows).cpu().numpy()
        for r, row in zip(who, logits):
            got[r].append(row)
        for r, _ in step:
            if at[r] == len(requests[r]):
                runner.release(live.pop(r))
    assert not live and all(at[r] == len(requests[r]) for r in requests)
    return {r: np.stack(v) for r, v in got.items()}


def portions(total, sizes):
    out, i = [], 0
    while total > 0:
        n = min(sizes[i % len(sizes)], total)
        out.append(n)
        total -= n
        i += 1
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(KAKUNEX))
def test_schedules_agree_with_plain(name, dtype, folders, plain_logits):
    """One sequence that passes every window several times: whole, decoded token by token behind a short prefix, and in
    portions of changing sizes down to two tokens and one, through a pool hardly larger than the request."""
    toks = tokens_for(name, 150, 1)
    want = plain_logits(name, toks)
    runner = make_runner(folders[name], dtype, 160, 2)
    seen = {}
    for label, cuts in (("whole", [150]), ("decode", [20] + [1] * 130), ("first token alone", [1, 149]),
                        ("portions", portions(150, [2, 3, 17, 64, 5, 2, 31, 1, 1]))):
        got = run_schedule(runner, {"a": toks}, [[("a", n)] for n in cuts])["a"]
        check_logits(got, want, dtype, f"{name} {label}")
        seen[label] = got
        assert runner.cache.idle
    if dtype == "float32":  # cuts change nothing beyond rounding
        for label, got in seen.items():
            assert np.abs(got - seen["whole"]).max() <= 2e-5 * np.abs(want).max(), label


@pytest.mark.parametrize("name", sorted(KAKUNEX))
def test_the_models_show_a_mask_that_is_off_by_one(name, folders, plain_logits):
    """What the comparison above is worth: with these weights a window or a run of kept keys that is one token off
    moves the logits by far more than the tolerance."""
    cfg, w = read_model_folder(folders[name])
    toks = tokens_for(name, 150, 1)
    want = plain_logits(name, toks)
    for i, layer in enumerate(cfg["layers"]):
        mask = layer["mixer"].get("left", {}).get("mask") if layer["type"] == "parallel" else None
        if not mask:
            continue
        for key in ("size", "keep_first"):
            if mask.get(key):
                off = copy.deepcopy(cfg)
                off["layers"][i]["mixer"]["left"]["mask"][key] -= 1
                assert np.abs(K.forward(off, w, toks) - want).max() > 50 * 1e-4 * np.abs(want).max(), (name, i, key)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(KAKUNEX))
def test_unequal_requests_in_one_batch_with_pages_and_slots_used_again(name, dtype, folders, plain_logits):
    """Five requests through three state slots and a pool that never holds them all: portions of some beside single
    tokens of others, a request of one token, requests admitted into slots and pages that others gave back."""
    lens = {"a": 150, "b": 37, "c": 1, "d": 70, "e": 33}
    reqs = {r: tokens_for(name, n, 10 + i) for i, (r, n) in enumerate(lens.items())}
    steps = [
        [("a", 29)], [("a", 2), ("b", 3)], [("a", 16), ("b", 30), ("c", 1)], [("a", 1), ("b", 1), ("d", 33)],
        [("a", 64), ("b", 1), ("d", 1)], [("b", 1), ("d", 2), ("a", 1)], [("b", 1), ("d", 30), ("a", 7)], [("a", 1), ("d", 1), ("e", 2)],
    ] + [[("a", 1), ("d", 1), ("e", 1)] for _ in range(3)] + [[("a", 26), ("e", 28)]]
    runner = make_runner(folders[name], dtype, 16 * 18, 3)
    got = run_schedule(runner, reqs, steps)
    assert runner.cache.idle
    for r in reqs:
        check_logits(got[r], plain_logits(name, reqs[r]), dtype, f"{name} request {r}")
    with pytest.raises(Exception):
        for _ in range(4):
            runner.acquire()


def test_long_decoding_through_a_small_pool(folders, plain_logits):
    """400 tokens one by one through 8 pages: the window's pages go round many times while the kept first pages stay."""
    name = "kxB"
    toks = tokens_for(name, 400, 7)
    runner = make_runner(folders[name], "float32", 16 * 8, 1)
    got = run_schedule(runner, {"a": toks}, [[("a", 1)] for _ in toks])["a"]
    check_logits(got, plain_logits(name, toks), "float32", "long decoding")
    assert runner.cache.idle


@pytest.mark.parametrize("name", sorted(KAKUNEX))
@pytest.mark.parametrize("chunk,graph", [(0, True), (16, True), (16, False)])
def test_greedy_generation_through_the_engine(name, chunk, graph, folders):
    from miniserve_amd.engine.engine import Engine
    from miniserve_amd.engine.request import SamplingParams
    from miniserve_amd.loading import load_model

    cfg, w = read_model_folder(folders[name])
    prompts = [tokens_for(name, n, 20 + n) for n in (1, 9, 40, 17, 26)]
    want = [K.greedy(cfg, w, p, 12) for p in prompts]
    eng = Engine(load_model(folders[name], "float32", DEV), kv_pool_tokens=16 * 14, max_running=3, chunked_prefill_size=chunk,
                 decode_graph=graph)
    assert eng.generate(prompts, SamplingParams(max_new_tokens=12)) == want
    assert eng.runner.cache.idle


def test_trace_replay(folders, plain_logits, tmp_path):
    from replay_util import Replay

    name = "kxA"
    a, b = tokens_for(name, 70, 31), tokens_for(name, 21, 32)
    with Replay(folders[name], "float32", tmp_path / "out", 128) as run:
        got = [run.step([("a", a[:33], [0, 32])]),
               run.step([("a", a[33:35], [1]), ("b", b, [20])], end=["b"]),
               run.step([("a", a[35:], [34])], end=["a"]),
               run.step([("c", b, [3, 20])], end=["c"])]
        assert run.close() == 0
    wa, wb = plain_logits(name, a), plain_logits(name, b)
    check_logits(np.concatenate(got), np.stack([wa[0], wa[32], wa[34], wb[20], wa[69], wb[3], wb[20]]), "float32", "trace replay")


def test_command_line_random_weights_generate_and_stress(tmp_path):
    """The command line serves the architecture like any other: a folder of random weights from the named preset,
    greedy generation from it against the plain implementation, and a sampled load that returns every page and slot."""
    import json
    import subprocess
    import sys

    from replay_util import ROOT

    folder = tmp_path / "m"
    run = lambda *a: subprocess.run([sys.executable, "-m", "miniserve_amd", *a], capture_output=True, text=True, cwd=str(ROOT), timeout=110)
    res = run("random-weights", "--preset", "kakunex-tiny", "--seed", "5", "--std", "0.1", "--norm-range", "0.6", "1.4", "--out", str(folder))
    assert res.returncode == 0, res.stderr[-2000:]
    cfg, w = read_model_folder(folder)
    prompt = np.random.default_rng(8).integers(0, cfg["vocab"], size=30).tolist()
    res = run("generate", "--model", str(folder), "--dtype", "float32", "--prompt-ids", ",".join(map(str, prompt)),
              "--max-new-tokens", "8", "--kv-pool-tokens", "256")
    assert res.returncode == 0, res.stderr[-2000:]
    assert json.loads(res.stdout.strip().splitlines()[-1])["outputs"] == [K.greedy(cfg, w, prompt, 8)]
    res = run("stress", "--model", str(folder), "--num-requests", "12", "--prompt-len", "4", "90", "--max-new-tokens", "1", "20",
              "--kv-pool-tokens", "640", "--max-running", "4", "--chunked-prefill-size", "64", "--temperature", "0.7", "--top-p", "0.9")
    assert res.returncode == 0, res.stdout[-1000:] + res.stderr[-2000:]
    report = json.loads(res.stdout.strip().splitlines()[-1])
    assert report["finished"] == 12 and report["idle"] and report["engine"]["architecture"] == "Kakunex"
