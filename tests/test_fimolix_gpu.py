"""Fimolix on the GPU against the plain implementation (``tests/plain/fimolix_plain.py``): every mechanism alone on
inputs made so that a fault shows, then whole models with random weights under every kind of schedule: whole
prompts, token-by-token decoding, portions down to two tokens, batches of unequal requests, pages and state slots
that are given back and used again, long decoding, greedy generation through the engine and its scheduler, and the
trace replay tool."""

from __future__ import annotations

import copy
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from fimolix_models import FIMOLIX, make_folder
from plain import fimolix_plain as F
from plain.model_folder import read_model_folder
from tolerances import check_logits

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
PAGE = 16


def ops():
    from miniserve_amd.kernels import ops as o

    o.library()
    return o


def dev(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV).contiguous()


def rounded(a, dtype):
    """What a kernel is given when ``a`` is stored in ``dtype``."""
    return dev(a, dtype).float().cpu().numpy().astype(np.float64)


def close(got, want, dtype, what="", tol=None):
    got = got.float().cpu().numpy().astype(np.float64)
    scale = max(float(np.abs(want).max()), 1e-30)
    tol = tol or (2e-5 if dtype == torch.float32 else 1.2e-2)
    worst = float(np.abs(got - want).max())
    assert worst <= tol * scale, f"{what}: max |diff| {worst:.3e} > {tol * scale:.3e}"


def step_batch(lens, starts, slots=None):
    """What the kernels read of a step: rows of ``lens`` new tokens behind ``starts`` cached ones."""
    pos = np.concatenate([np.arange(s, s + n) for n, s in zip(lens, starts)])
    row = np.concatenate([np.full(n, i) for i, n in enumerate(lens)])
    flat = np.arange(int(sum(lens)))
    single = np.concatenate([np.full(n, n == 1) for n in lens])
    n_dec = int(single.sum())
    mixed = 0 < n_dec < len(flat)
    b = SimpleNamespace(num_rows=len(lens), num_tokens=int(sum(lens)), positions=dev(pos, torch.int32), token_row=dev(row, torch.int32),
                        row_start=dev(np.concatenate(([0], np.cumsum(lens))), torch.int32), starts=dev(starts, torch.int32),
                        state_slots=dev(slots if slots is not None else list(range(len(lens))), torch.int32),
                        num_decode_tokens=n_dec, decode_tokens=dev(flat[single], torch.int32) if mixed else None,
                        prefill_tokens=dev(flat[~single], torch.int32) if mixed else None,
                        max_kv_len=max(s + n for n, s in zip(lens, starts)), row_lens=list(lens), row_starts_host=list(starts), memo={})
    b.is_decode = n_dec == len(flat)
    return b


# ---------------------------------------------------------------- mechanisms alone


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [1, 1000, 4099])
def test_activation_without_a_gate(n, dtype):
    x = np.random.default_rng(n).normal(size=(3, n)) * 3
    close(ops().activate(dev(x), "gelu_tanh", dtype), F.gelu_tanh(x), dtype)
    with pytest.raises(NotImplementedError):
        ops().activate(dev(x), "swiglu_clamped", dtype)


@pytest.mark.parametrize("width", [5, 176, 600])
def test_norm_of_a_sublayers_output_into_the_stream(width):
    """``residual += y / rms(y) * w`` with ``y`` a stream, a stream plus partial sums of its last product, or partial sums
    alone."""
    rng = np.random.default_rng(width)
    r, y, w = rng.normal(size=(6, width)), rng.normal(size=(6, width)) * 10, rng.normal(size=width) + 1
    parts = rng.normal(size=(3, 6, width))
    for stream, pending, total in ((y, None, y), (y, parts, y + parts.sum(0)), (None, parts, parts.sum(0))):
        res = dev(r)
        ops().normed_add(res, None if stream is None else dev(stream), dev(w), 1e-6, None if pending is None else ops().SplitSum(dev(pending)))
        close(res, r + F.rms_norm(total, w, 1e-6), torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,size", [(1, 1), (3, 7), (6, 80)])
def test_gate_per_head(heads, size, dtype):
    rng = np.random.default_rng(heads)
    o, x = rng.normal(size=(5, heads * size)), rng.normal(size=(5, heads + 9)) * 3
    want = (rounded(o, dtype).reshape(5, heads, size) * F.sigmoid(x[:, 4 : 4 + heads])[:, :, None]).reshape(5, -1)
    close(ops().head_gate_(dev(o, dtype), dev(x), 4, heads), want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("groups,per,size", [(1, 1, 5), (2, 3, 24), (3, 1, 96), (1, 4, 130)])
def test_difference_of_two_maps(groups, per, size, dtype):
    rng = np.random.default_rng(size)
    a = rng.normal(size=(4, groups, 2, per, size))
    a[0] *= 1e-4  # small against eps = 1e-3: eps under the root matters
    lam, eps, scale = 0.7, 1e-3, 0.4
    ar = rounded(a, dtype)
    o = ar[:, :, 0] - lam * ar[:, :, 1]  # [T, groups, per, size]: head = group * per + its place in the group
    want = (F.unit_rms(o, eps) * scale).reshape(4, -1)
    got = ops().map_difference_norm(dev(a.reshape(4, -1), dtype), groups, per, size, lam, eps, scale)
    close(got, want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,k,n,stride,col", [(3, 5, 7, 11, 2), (2, 32, 64, 80, 0), (4, 64, 24, 24, 0), (1, 8, 8, 16, 8), (2, 128, 40, 48, 8)])
def test_product_per_head(heads, k, n, stride, col, dtype):
    """Strided in place where every slice starts at a multiple of 16 bytes, through copies where not; the columns of
    ``out`` that no head writes stay as they were."""
    rng = np.random.default_rng(k)
    for m in (1, 5, 150):
        x, w = rng.normal(size=(m, heads * k)), rng.normal(size=(heads, n, k))
        out = torch.full((m, heads * stride), 7.0, dtype=dtype, device=DEV)
        ops().head_linear(dev(x, dtype), dev(w, dtype), out, col)
        xr, wr = rounded(x, dtype), rounded(w, dtype)
        want = np.full((m, heads, stride), 7.0)
        for h in range(heads):
            want[:, h, col : col + n] = xr[:, h * k : (h + 1) * k] @ wr[h].T
        close(out, want.reshape(m, -1), dtype, f"{m} rows", tol=2e-5 if dtype == torch.float32 else 8e-3)
        if col == 0 and stride == n:  # with a gate per head in the product's epilogue (or behind it)
            g = rng.normal(size=(m, heads + 3)) * 2
            gated = torch.empty((m, heads * n), dtype=dtype, device=DEV)
            ops().head_linear(dev(x, dtype), dev(w, dtype), gated, 0, gate=(dev(g), 2))
            close(gated, (want * F.sigmoid(g[:, 2 : 2 + heads])[:, :, None]).reshape(m, -1), dtype, f"{m} rows, gated",
                  tol=2e-5 if dtype == torch.float32 else 8e-3)


def conv_setup(rng, gq, gk, hv, d, dv, taps, dtype, norm=True):
    c = (gq + gk) * d + hv * dv
    cw = rng.normal(size=(c, taps))
    qw, kw = (rng.normal(size=d) + 1, rng.normal(size=d) + 1) if norm else (None, None)
    pages = 12
    kc = torch.zeros((pages + 1, gk, PAGE, d), dtype=dtype, device=DEV)
    vc = torch.zeros((pages + 1, hv, dv, PAGE), dtype=dtype, device=DEV)
    return c, cw, qw, kw, kc, vc


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("gq,gk,hv,d,dv,taps", [(4, 2, 1, 8, 12, 4), (6, 2, 2, 5, 3, 2), (2, 2, 1, 70, 9, 5), (2, 2, 2, 16, 16, 1)])
def test_short_convolution_norm_and_store(gq, gk, hv, d, dv, taps, dtype):
    """A sequence cut into steps of every kind (one token, fewer tokens than the state holds, more), in a state slot
    that holds another request's leftovers, beside a second request; keys and values land in the pages at their slots."""
    o = ops()
    rng = np.random.default_rng(taps * 100 + d)
    c, cw, qw, kw, kc, vc = conv_setup(rng, gq, gk, hv, d, dv, taps, dtype)
    T, eps = 40, 1e-5
    u = {r: rng.normal(size=(T, c)) for r in "ab"}
    cwr = rounded(cw, dtype)
    want = {}
    for r in "ab":
        y = F.short_conv(u[r], cwr)
        q = F.rms_norm(y[:, : gq * d].reshape(T, gq, d), rounded(qw, dtype), eps).reshape(T, -1)
        k = F.rms_norm(y[:, gq * d : (gq + gk) * d].reshape(T, gk, d), rounded(kw, dtype), eps)
        want[r] = (q, k, y[:, (gq + gk) * d :].reshape(T, hv, dv))
    state = torch.full((4, max(taps - 1, 1), c), 50.0, device=DEV) if taps > 1 else None  # leftovers: must not be read at position 0
    slot_of = {"a": 2, "b": 0}
    pages_of = {"a": [5, 1, 9], "b": [0, 7, 3]}
    at = {"a": 0, "b": 0}
    got_q = {"a": [], "b": []}
    for step in ([("a", 1)], [("a", 2), ("b", 7)], [("a", 1), ("b", 1)], [("b", 2), ("a", 9)], [("a", 1), ("b", 30)], [("a", 26)]):
        lens, starts = [n for _, n in step], [at[r] for r, _ in step]
        b = step_batch(lens, starts, [slot_of[r] for r, _ in step])
        x = np.concatenate([u[r][at[r] : at[r] + n] for r, n in step])
        slots = np.concatenate([[pages_of[r][p // PAGE] * PAGE + p % PAGE for p in range(at[r], at[r] + n)] for r, n in step])
        q = o.conv_norm_store(dev(x), dev(cw, dtype), taps, state, b, dev(qw, dtype), dev(kw, dtype), eps, dev(slots, torch.int32), kc, vc,
                              gq, gk, hv, d, dv, dtype).float().cpu().numpy()
        i = 0
        for r, n in step:
            got_q[r].append(q[i : i + n])
            i += n
            at[r] += n
    for r in "ab":
        q, k, v = want[r]
        close(torch.tensor(np.concatenate(got_q[r])), q, dtype, f"queries of {r}")
        kk = torch.stack([kc[pages_of[r][p // PAGE], :, p % PAGE] for p in range(T)])
        vv = torch.stack([vc[pages_of[r][p // PAGE], :, :, p % PAGE] for p in range(T)])
        close(kk, k, dtype, f"keys of {r}")
        close(vv, v, dtype, f"values of {r}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pairing", ["adjacent", "halves"])
@pytest.mark.parametrize("heads,dn,r,c,rot", [(3, 8, 8, 24, 4), (2, 5, 6, 9, 6), (1, 32, 16, 300, 16), (2, 4, 2, 3, 0)])
def test_latent_preparation(heads, dn, r, c, rot, pairing, dtype):
    o = ops()
    rng = np.random.default_rng(c)
    T, eps, base = 9, 1e-5, 50.0
    q_col, kv_col = 3, 3 + heads * (dn + r) + 2
    x = rng.normal(size=(T, kv_col + c + r + 4))
    pos = np.array([0, 1, 2, 700, 701, 5, 6, 7, 33])
    cw = rng.normal(size=c) + 1
    f = base ** (-2.0 * np.arange(rot // 2) / max(rot, 1))
    ang = pos[:, None] * f
    table = np.concatenate((np.cos(ang), np.sin(ang)), axis=1)

    def turn(v):  # [T, ..., r]
        out = v.copy()
        if not rot:
            return out
        cs = table.reshape((T,) + (1,) * (v.ndim - 2) + (rot,))
        co, si = cs[..., : rot // 2], cs[..., rot // 2 :]
        a, b = (v[..., 0:rot:2], v[..., 1:rot:2]) if pairing == "adjacent" else (v[..., : rot // 2], v[..., rot // 2 : rot])
        ra, rb = a * co - b * si, b * co + a * si
        if pairing == "adjacent":
            out[..., 0:rot:2], out[..., 1:rot:2] = ra, rb
        else:
            out[..., : rot // 2], out[..., rot // 2 : rot] = ra, rb
        return out

    if pairing == "adjacent" and rot:  # the same turn as the plain implementation's
        assert np.allclose(turn(x[:, kv_col + c : kv_col + c + r]), F.rotate_adjacent(x[:, kv_col + c : kv_col + c + r], pos, rot, base))
    slots = rng.permutation(5 * PAGE)[:T]
    kc = torch.zeros((6, 1, PAGE, c + r), dtype=dtype, device=DEV)
    vc = torch.zeros((6, 1, c, PAGE), dtype=dtype, device=DEV)
    qp, qf = o.latent_prepare(dev(x), q_col, kv_col, dev(table) if rot else None, rot, pairing, dev(cw, dtype), eps,
                              dev(slots, torch.int32), kc, vc, heads, dn, r, c, dtype)
    q = x[:, q_col : q_col + heads * (dn + r)].reshape(T, heads, dn + r)
    close(qp, q[:, :, :dn].reshape(T, -1), dtype, "plain query parts")
    close(qf.view(T, heads, c + r)[:, :, c:], turn(q[:, :, dn:]), dtype, "turned query parts")
    rows = kc.view(-1, c + r)[dev(slots, torch.int64)]
    close(rows[:, :c], F.rms_norm(x[:, kv_col : kv_col + c], rounded(cw, dtype), eps), dtype, "latent")
    close(rows[:, c:], turn(x[:, kv_col + c : kv_col + c + r]), dtype, "shared key part")
    values = vc[:, 0].permute(0, 2, 1).reshape(-1, c)[dev(slots, torch.int64)]  # the latent once more, tokens side by side
    assert torch.equal(values, rows[:, :c])
    # a layer that keeps nothing: queries only, the cache stays as it is
    before = kc.clone()
    o.latent_prepare(dev(x), q_col, None, dev(table) if rot else None, rot, pairing, None, eps, None, None, None, heads, dn, r, c, dtype)
    assert torch.equal(kc, before)


def plain_attention(q, k, v, scale, size, cap, sinks, k_of, v_of):
    """``q [T, Hq, D]``, ``k [T, Hk, D]``, ``v [T, Hv, E]`` of one sequence; query head a reads key head ``k_of(a)`` and value
    head ``v_of(a)``; float64."""
    T, H, _ = q.shape
    out = np.zeros((T, H, v.shape[2]))
    for a in range(H):
        s = (q[:, a] @ k[:, k_of(a)].T) * scale
        if cap:
            s = cap * np.tanh(s / cap)
        seen = F.sliding(T, size) if size else F.causal(T)
        out[:, a] = F.masked_softmax(s, seen, None if sinks is None else float(sinks[a])) @ v[:, v_of(a)]
    return out


def run_attention(o, q, kc, vc, pages, cuts, T, **kw):
    """The sequence's queries in steps of ``cuts`` tokens over the pages it holds."""
    table = dev([pages + [0] * (-len(pages) % 4)], torch.int32)
    got, at = [], 0
    for n in cuts:
        n = min(n, T - at)
        if n <= 0:
            break
        b = step_batch([n], [at])
        got.append(o.paged_attention(q[at : at + n].contiguous(), kc, vc, table, b, **kw))
        at += n
    return torch.cat(got)


CUTS = ([400], [150] + [1] * 250, [2, 3, 64, 5, 2, 31, 1, 1, 190, 1, 100])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hq,hk,share,d,e,cap", [(8, 4, 2, 16, 24, 4.0), (6, 2, 2, 10, 6, 30.0), (4, 4, 2, 64, 64, 0.0), (2, 2, 1, 40, 72, 2.0),
                                                 (8, 4, 2, 128, 256, 4.0), (4, 2, 2, 32, 48, 3.0), (16, 2, 2, 96, 32, 0.0)])
def test_capped_scores_and_shared_values(hq, hk, share, d, e, cap, dtype):
    """Several key heads weigh one value head; scores are bounded. One far key per query head is made to stand out
    (beyond the cap's linear range), so that a lost key, a wrong head pairing or a missing cap moves the result."""
    o = ops()
    rng = np.random.default_rng(hq * d)
    T, scale = 400, 0.3
    q, k, v = rng.normal(size=(T, hq, d)), rng.normal(size=(T, hk, d)), rng.normal(size=(T, hk // share, e))
    for a in range(hq):
        far = 3 + 5 * a  # a key far back, close to a page's border for some heads
        k[far, a // (hq // hk)] = q[T - 1, a] * 3
    qr, kr, vr = rounded(q, dtype), rounded(k, dtype), rounded(v, dtype)
    want = plain_attention(qr, kr, vr, scale, 0, cap, None, lambda a: a // (hq // hk), lambda a: a // (hq // hk) // share)
    assert cap == 0 or np.abs(plain_attention(qr, kr, vr, scale, 0, 0.0, None, lambda a: a // (hq // hk), lambda a: a // (hq // hk) // share) - want).max() > 0.05
    pages = list(rng.permutation(30)[: -(-T // PAGE)])
    kc = torch.zeros((31, hk, PAGE, d), dtype=dtype, device=DEV)
    vc = torch.zeros((31, hk // share, e, PAGE), dtype=dtype, device=DEV)
    for p in range(T):
        kc[pages[p // PAGE], :, p % PAGE] = dev(k[p], dtype)
        vc[pages[p // PAGE], :, :, p % PAGE] = dev(v[p], dtype)
    for cuts in CUTS:
        got = run_attention(o, dev(q.reshape(T, -1), dtype), kc, vc, [int(p) for p in pages], cuts, T, num_heads=hq, num_kv_heads=hk,
                            head_dim=d, scale=scale, window=0, value_dim=e, softcap=cap, value_share=share)
        close(got, want.reshape(T, -1), dtype, f"cuts {cuts[:3]}", tol=2e-5 if dtype == torch.float32 else 6e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("inside", [True, False])
@pytest.mark.parametrize("h,d,e,size", [(3, 32, 24, 37), (2, 11, 9, 16), (2, 288, 272, 100), (4, 40, 40, 0), (1, 192, 160, 80),
                                        (16, 192, 160, 80), (8, 576, 512, 150), (12, 64, 48, 20), (40, 96, 64, 70)])
def test_sinks_a_window_and_values_that_repeat_the_keys(h, d, e, size, inside, dtype):
    """One key head whose rows' first elements are also the values (read from the key rows themselves, or from a value
    cache that repeats them), a window, a sink per head. The key just inside the window of the last query and the one
    just outside are made to stand out: a window one token off shows. Pages that the window has passed are given away
    (their table entries are no pages)."""
    o = ops()
    rng = np.random.default_rng(h * d)
    T, scale = 400, 0.25
    q, k = rng.normal(size=(T, h, d)), rng.normal(size=(T, 1, d))
    if size:
        k[T - size, 0] = q[T - 1].mean(0) * 2      # just inside
        k[T - size - 1, 0] = q[T - 1].mean(0) * 4  # just outside
    sinks = rng.normal(size=h) * 2 + 1
    qr, kr = rounded(q, dtype), rounded(k, dtype)
    want = plain_attention(qr, kr, kr[:, :, :e], scale, size, 0.0, sinks, lambda a: 0, lambda a: 0)
    none = plain_attention(qr, kr, kr[:, :, :e], scale, size, 0.0, None, lambda a: 0, lambda a: 0)
    assert np.abs(none - want).max() > 0.05 * np.abs(want).max()
    pages = [int(p) for p in rng.permutation(30)[: -(-T // PAGE)]]
    kc = torch.zeros((31, 1, PAGE, d), dtype=dtype, device=DEV)
    vc = None if inside else torch.zeros((31, 1, e, PAGE), dtype=dtype, device=DEV)
    for p in range(T):
        kc[pages[p // PAGE], 0, p % PAGE] = dev(k[p, 0], dtype)
        if not inside:
            vc[pages[p // PAGE], 0, :, p % PAGE] = dev(k[p, 0, :e], dtype)
    kw = dict(num_heads=h, num_kv_heads=1, head_dim=d, scale=scale, window=size, value_dim=e, sinks=dev(sinks), values_in_keys=inside)
    for cuts in CUTS:
        got = run_attention(o, dev(q.reshape(T, -1), dtype), kc, vc, pages, cuts, T, **kw)
        close(got, want.reshape(T, -1), dtype, f"cuts {cuts[:3]}", tol=2e-5 if dtype == torch.float32 else 6e-3)
    if size:  # the last tokens again, with every page before the window gone
        first_live = (T - 20 - size + 1) // PAGE
        gone = [-1 if i < first_live else p for i, p in enumerate(pages)]
        table = dev([gone + [0] * (-len(gone) % 4)], torch.int32)
        b = step_batch([20], [T - 20])
        got = o.paged_attention(dev(q.reshape(T, -1), dtype)[T - 20 :].contiguous(), kc, vc, table, b, **kw)
        close(got, want.reshape(T, -1)[T - 20 :], dtype, "pages before the window given away", tol=2e-5 if dtype == torch.float32 else 6e-3)


def test_unequal_rows_in_one_attention_step():
    """Rows of one token beside rows of several in one launch pair: each row's result is what it is alone."""
    o = ops()
    rng = np.random.default_rng(5)
    h, d, e, size = 3, 24, 16, 20
    lens, starts = [1, 7, 1, 30], [50, 0, 3, 41]
    total = [s + n for s, n in zip(starts, lens)]
    seqs = [(rng.normal(size=(t, h, d)), rng.normal(size=(t, 1, d))) for t in total]
    sinks = rng.normal(size=h)
    kc = torch.zeros((40, 1, PAGE, d), dtype=torch.float32, device=DEV)
    tables, free = [], list(rng.permutation(39))
    for (q, k), t in zip(seqs, total):
        pages = [int(free.pop()) for _ in range(-(-t // PAGE))]
        for p in range(t):
            kc[pages[p // PAGE], 0, p % PAGE] = dev(k[p, 0])
        tables.append(pages + [0] * (8 - len(pages)))
    b = step_batch(lens, starts)
    qs = np.concatenate([q[s:].reshape(n, -1) for (q, _), s, n in zip(seqs, starts, lens)])
    got = o.paged_attention(dev(qs), kc, None, dev(tables, torch.int32), b, h, 1, d, 0.3, size, e, sinks=dev(sinks), values_in_keys=True)
    want = np.concatenate([plain_attention(q, k, k[:, :, :e], 0.3, size, 0.0, sinks, lambda a: 0, lambda a: 0)[s:].reshape(n, -1)
                           for (q, k), s, n in zip(seqs, starts, lens)])
    close(got, want, torch.float32)


# ---------------------------------------------------------------- whole models


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("fimolix")
    return {name: make_folder(root, name) for name in FIMOLIX}


@pytest.fixture(scope="module")
def plain_logits(folders):
    memo = {}

    def get(name, tokens):
        key = (name, tuple(tokens))
        if key not in memo:
            cfg, w = read_model_folder(folders[name])
            memo[key] = F.forward(cfg, w, tokens)
        return memo[key]

    return get


def tokens_for(name, n, seed):
    return np.random.default_rng(seed).integers(0, FIMOLIX[name][0]["vocab"], size=n).tolist()


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
@pytest.mark.parametrize("name", sorted(FIMOLIX))
def test_schedules_agree_with_plain(name, dtype, folders, plain_logits):
    """One sequence that passes every window several times: whole, decoded token by token behind a short prefix, and in
    portions of changing sizes down to two tokens and one, through a pool hardly larger than the request."""
    toks = tokens_for(name, 150, 1)
    want = plain_logits(name, toks)
    runner = make_runner(folders[name], dtype, 160, 2)
    seen = {}
    for label, cuts in (("whole", [150]), ("decode", [20] + [1] * 130), ("first token alone", [1, 149]), ("two, then one by one", [2] + [1] * 148),
                        ("portions", portions(150, [2, 3, 17, 64, 5, 2, 31, 1, 1]))):
        got = run_schedule(runner, {"a": toks}, [[("a", n)] for n in cuts])["a"]
        check_logits(got, want, dtype, f"{name} {label}")
        seen[label] = got
        assert runner.cache.idle
    if dtype == "float32":  # cuts change nothing beyond rounding
        for label, got in seen.items():
            assert np.abs(got - seen["whole"]).max() <= 2e-5 * np.abs(want).max(), label


@pytest.mark.parametrize("name", sorted(FIMOLIX))
def test_the_models_show_what_is_left_out(name, folders, plain_logits):
    """What the comparison above is worth: with these weights a window one token off, a sink left out, a cap or a
    weight of the second map that is wrong, a convolution tap lost or a borrowed cache that is the layer's own moves the
    logits by far more than the tolerance."""
    cfg, w = read_model_folder(folders[name])
    toks = tokens_for(name, 150, 1)
    want = plain_logits(name, toks)
    floor = 50 * 1e-4 * np.abs(want).max()

    def moved(c=cfg, weights=w):
        return np.abs(F.forward(c, weights, toks) - want).max()

    for i, layer in enumerate(cfg["layers"]):
        m = layer["mixer"]
        off = copy.deepcopy(cfg)
        mo = off["layers"][i]["mixer"]
        if layer["type"] == "latent_attention":
            if m.get("mask"):
                mo["mask"]["size"] -= 1
                assert moved(off) > floor, (name, i, "window")
            no_sink = dict(w)
            no_sink[f"l{i}.mix.sink"] = w[f"l{i}.mix.sink"] - 60.0
            assert moved(weights=no_sink) > floor, (name, i, "sink")
            if m.get("kv_from") is not None:
                turned = dict(w)
                src = m["kv_from"]
                turned[f"l{src}.mix.dkv"] = w[f"l{src}.mix.dkv"][::-1].copy()  # another latent: the reader must notice
                assert moved(weights=turned) > floor, (name, i, "borrowed cache")
        else:
            if m.get("softcap"):
                mo["softcap"] *= 2
                assert moved(off) > floor, (name, i, "cap")
                mo["softcap"] /= 2
            mo["diff"] += 0.05
            assert moved(off) > floor, (name, i, "second map's weight")
            if m["conv"] > 1:
                lost = dict(w)
                lost[f"l{i}.mix.k.conv"] = w[f"l{i}.mix.k.conv"].copy()
                lost[f"l{i}.mix.k.conv"][:, 0] = 0.0  # the oldest tap
                assert moved(weights=lost) > floor, (name, i, "oldest tap")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(FIMOLIX))
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
    """300 tokens one by one: the windowed groups' pages go round many times, the convolution's state moves on with
    every token, and the groups that keep every token fill the pool to its last page."""
    name = "fxB"
    toks = tokens_for(name, 300, 7)
    runner = make_runner(folders[name], "float32", 16 * 19, 1)
    got = run_schedule(runner, {"a": toks}, [[("a", 1)] for _ in toks])["a"]
    check_logits(got, plain_logits(name, toks), "float32", "long decoding")
    assert runner.cache.idle


def test_a_borrowed_cache_is_kept_as_long_as_its_widest_reader_needs(folders):
    from miniserve_amd.loading import load_model
    from miniserve_amd.engine.runner import ModelRunner

    for name, window in (("fxA", 33), ("fxB", 21), ("fxD", 40)):
        runner = ModelRunner(load_model(folders[name], "float32", DEV), kv_pool_tokens=64, max_running=1)
        layers = FIMOLIX[name][0]["layers"]
        latent = [g for g in runner.layout.groups if layers[g.slots[0]]["type"] == "latent_attention"]
        assert [g.window for g in latent] == [window], name
        assert len(latent[0].slots) == 1  # the reader has no pages of its own


@pytest.mark.parametrize("name", sorted(FIMOLIX))
@pytest.mark.parametrize("chunk,graph", [(0, True), (16, True), (16, False)])
def test_greedy_generation_through_the_engine(name, chunk, graph, folders):
    from miniserve_amd.engine.engine import Engine
    from miniserve_amd.engine.request import SamplingParams
    from miniserve_amd.loading import load_model

    cfg, w = read_model_folder(folders[name])
    prompts = [tokens_for(name, n, 20 + n) for n in (1, 9, 40, 17, 26)]
    want = [F.greedy(cfg, w, p, 12) for p in prompts]
    eng = Engine(load_model(folders[name], "float32", DEV), kv_pool_tokens=16 * 14, max_running=3, chunked_prefill_size=chunk,
                 decode_graph=graph)
    assert eng.generate(prompts, SamplingParams(max_new_tokens=12)) == want
    assert eng.runner.cache.idle


def test_trace_replay(folders, plain_logits, tmp_path):
    from replay_util import Replay

    name = "fxA"
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
    res = run("random-weights", "--preset", "fimolix-tiny", "--seed", "5", "--std", "0.1", "--norm-range", "0.6", "1.4", "--out", str(folder))
    assert res.returncode == 0, res.stderr[-2000:]
    cfg, w = read_model_folder(folder)
    prompt = np.random.default_rng(8).integers(0, cfg["vocab"], size=30).tolist()
    res = run("generate", "--model", str(folder), "--dtype", "float32", "--prompt-ids", ",".join(map(str, prompt)),
              "--max-new-tokens", "8", "--kv-pool-tokens", "256")
    assert res.returncode == 0, res.stderr[-2000:]
    assert json.loads(res.stdout.strip().splitlines()[-1])["outputs"] == [F.greedy(cfg, w, prompt, 8)]
    res = run("stress", "--model", str(folder), "--num-requests", "12", "--prompt-len", "4", "90", "--max-new-tokens", "1", "20",
              "--kv-pool-tokens", "640", "--max-running", "4", "--chunked-prefill-size", "64", "--temperature", "0.7", "--top-p", "0.9")
    assert res.returncode == 0, res.stdout[-1000:] + res.stderr[-2000:]
    report = json.loads(res.stdout.strip().splitlines()[-1])
    assert report["finished"] == 12 and report["idle"] and report["engine"]["architecture"] == "Fimolix"
