"""Zederax on the GPU: every kernel of its layers against the plain implementation's function of the same mechanism,
then whole models through the step function, ``bin/trace_run`` and the engine's own entry point, in 32-bit and bfloat16."""
import math
import os

import numpy as np
import pytest
import torch

import plain_zederax as Z
import traces as TR
from helpers import make_meta, random_block_tables
from zederax_configs import ZED

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def K():
    from levanter_amd.kernels import get_kernels

    return get_kernels()


def tol(dtype, f32=2e-5, bf16=2e-2):
    return dict(rtol=f32, atol=f32) if dtype == torch.float32 else dict(rtol=bf16, atol=bf16)


def as_bf16_numbers(x):
    return x.to(torch.bfloat16).double()


# ------------------------------------------------------------------------------------------------ kernels
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(5, 3, 2, 24, 8), (130, 4, 4, 64, 128), (1, 1, 1, 8, 200)])
def test_unit_norm_of_heads_and_blend_of_values(dtype, shape):
    T, H, G, dk, dv = shape
    g = torch.Generator().manual_seed(T)
    width = (H + G) * dk + G * dv + 8
    p = as_bf16_numbers(torch.randn(T, width, generator=g) * 3)
    first = as_bf16_numbers(torch.randn(T, G * dv + 16, generator=g))
    lam = torch.tensor([0.3125])
    buf = p.to(dtype).to(DEV)
    fbuf = first.to(dtype).to(DEV)
    v = buf[:, (H + G) * dk:(H + G) * dk + G * dv]
    K().head_prepare(buf[:, :(H + G) * dk], H + G, dk, 1e-5, v=v, v_first=fbuf[:, 8:8 + G * dv], n_blend=G, value_dim=dv, blend=lam.to(DEV))
    want_qk = Z.unit_rms(p[:, :(H + G) * dk].view(T, H + G, dk), 1e-5).reshape(T, -1)
    want_v = Z.blend_values(p[:, (H + G) * dk:(H + G) * dk + G * dv], first[:, 8:8 + G * dv], lam.double())
    got = buf.cpu().double()
    torch.testing.assert_close(got[:, :(H + G) * dk], want_qk, **tol(dtype))
    torch.testing.assert_close(got[:, (H + G) * dk:-8], want_v, **tol(dtype))
    assert torch.equal(got[:, -8:], p[:, -8:])  # columns behind the heads are not touched
    # each half alone
    buf2 = p.to(dtype).to(DEV)
    K().head_prepare(buf2[:, :H * dk], H, dk, 1e-5)
    torch.testing.assert_close(buf2.cpu().double()[:, :H * dk], want_qk[:, :H * dk], **tol(dtype))
    assert torch.equal(buf2.cpu().double()[:, H * dk:], p[:, H * dk:])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(5, 3, 1, 24, 8), (9, 4, 2, 64, 128), (1, 2, 2, 8, 16)])
@pytest.mark.parametrize("blend", [True, False])
def test_single_tokens_are_prepared_and_written_by_one_kernel(dtype, shape, blend):
    """Unit norms, the blend and the write into the pages in one kernel, against the plain functions, with a token that is
    written nowhere; the pages hold what the two separate kernels write."""
    from emulated_kernels import EmulatedKernels

    T, H, G, dk, dv = shape
    ps, n_pages = 16, 6
    g = torch.Generator().manual_seed(T + dk)
    q = as_bf16_numbers(torch.randn(T, H * dk, generator=g))
    k = as_bf16_numbers(torch.randn(T, G * dk, generator=g))
    v = as_bf16_numbers(torch.randn(T, G * dv, generator=g))
    first = as_bf16_numbers(torch.randn(T, G * dv, generator=g))
    lam = torch.tensor([0.625])
    dest = (torch.randperm(n_pages * ps, generator=g)[:T]).to(torch.int32)
    if T > 2:
        dest[1] = -1
    qd, kd, vd_, fd = (t.to(dtype).to(DEV) for t in (q, k, v, first))
    kp = torch.zeros(n_pages, G * dk * ps, dtype=dtype, device=DEV)
    vp = torch.zeros(n_pages, G * dv * ps, dtype=dtype, device=DEV)
    K().head_prepare_write(qd, kd, vd_, kp, vp, dest.to(DEV), H, G, dk, dv, ps, 1e-5, v_first=fd if blend else None, blend=lam.to(DEV) if blend else None)
    want_q = Z.unit_rms(q.view(T, H, dk), 1e-5).reshape(T, -1)
    want_k = Z.unit_rms(k.view(T, G, dk), 1e-5)
    want_v = Z.blend_values(v, first if blend else None, lam.double()).view(T, G, dv)
    torch.testing.assert_close(qd.cpu().double(), want_q, **tol(dtype))
    kv = EmulatedKernels.k_view(kp.cpu().double(), G, dk, ps)
    vv = EmulatedKernels.v_view(vp.cpu().double(), G, dv, ps)
    for t in range(T):
        d = int(dest[t])
        if d < 0:
            continue
        torch.testing.assert_close(kv[d // ps, :, :, d % ps, :].reshape(G, dk), want_k[t], **tol(dtype))
        torch.testing.assert_close(vv[d // ps, :, :, d % ps], want_v[t], **tol(dtype))
    written = sum(1 for t in range(T) if int(dest[t]) >= 0)
    assert int((kp != 0).sum()) <= written * G * dk and int((vp != 0).sum()) <= written * G * dv  # nothing else is touched
    # the two separate kernels leave the same bits
    q2, k2, v2 = (t.to(dtype).to(DEV) for t in (q, k, v))
    qk = torch.cat([q2, k2], 1)
    K().head_prepare(qk, H + G, dk, 1e-5, v=v2 if blend else None, v_first=fd if blend else None, n_blend=G if blend else 0, value_dim=dv,
                     blend=lam.to(DEV) if blend else None)
    kp2, vp2 = torch.zeros_like(kp), torch.zeros_like(vp)
    K().kv_write(qk[:, H * dk:], v2, kp2, vp2, dest.to(DEV), G, dk, ps, value_dim=dv)
    assert torch.equal(kp, kp2) and torch.equal(vp, vp2) and torch.equal(qd, qk[:, :H * dk])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,F", [(3, 40), (70, 1000), (2, 8200)])
def test_polynomial_activation_with_normed_powers(dtype, T, F):
    g = torch.Generator().manual_seed(F)
    z = as_bf16_numbers(torch.randn(T, F + 8, generator=g) * 2)
    c = torch.tensor([0.7, -1.3, 0.45, 0.2])
    zb = z.to(dtype).to(DEV)
    out = torch.zeros(T, F + 4, dtype=dtype, device=DEV)
    K().poly_norm(zb[:, :F], c.to(DEV), 1e-6, out[:, :F])
    want = Z.poly_norm(z[:, :F], c.double(), 1e-6)
    torch.testing.assert_close(out.cpu().double()[:, :F], want, **tol(dtype, bf16=3e-2))
    assert not out[:, F:].any()
    K().poly_norm(zb[:, :F], c.to(DEV), 1e-6, zb[:, :F])  # in place, as the feed-forward calls it
    torch.testing.assert_close(zb.cpu().double()[:, :F], want, **tol(dtype, bf16=3e-2))


@pytest.mark.parametrize("T,D", [(7, 64), (3, 30), (129, 257), (1, 1)])
def test_weighted_sum_of_all_results_so_far(T, D):
    g = torch.Generator().manual_seed(D)
    n_runs = 5
    results = [torch.randn(T, D, generator=g) for _ in range(n_runs + 1)]
    streams = torch.full((n_runs + 1, T, D), float("nan"), device=DEV)
    streams[0] = results[0].to(DEV)
    for i in range(n_runs):
        w = torch.randn(i + 2, generator=g)
        x = results[i + 1].clone().to(DEV)
        K().stream_average(streams, x, w.to(DEV), i + 2)
        want = Z.depth_average([r.double() for r in results[:i + 2]], w.double())
        torch.testing.assert_close(x.cpu().double(), want, rtol=1e-5, atol=1e-5)
        assert torch.equal(streams[i + 1].cpu(), results[i + 1])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,D", [(7, 64), (3, 30), (40, 1000)])
def test_weighted_sum_inside_the_norm_that_reads_it(dtype, T, D):
    """The deferred sum: computed by the norm's kernel, stored as the separate kernel stores it; with a selection of rows
    (one named twice) only the normed rows come out."""
    g = torch.Generator().manual_seed(D + 1)
    n = 4
    results = [torch.randn(T, D, generator=g) for _ in range(n)]
    w, nw = torch.randn(n, generator=g), 1 + 0.2 * torch.randn(D, generator=g)
    want_x = Z.depth_average([r.double() for r in results], w.double())
    want_h = Z.rms_norm(want_x, nw.double(), 1e-5)
    for rows in (None, torch.tensor([T - 1, 0, T - 1], dtype=torch.int32)):
        streams = torch.zeros(n + 2, T, D, device=DEV)
        for j in range(n - 1):
            streams[j] = results[j].to(DEV)
        x = results[n - 1].clone().to(DEV)
        pending = K().stream_average(streams, x, w.to(DEV), n, defer=True)
        assert pending is not None and torch.equal(x.cpu(), results[n - 1])  # nothing has run yet
        out = torch.empty(T if rows is None else 3, D, dtype=dtype, device=DEV)
        K().norm(x, nw.to(DEV), None, 1e-5, out, rows=None if rows is None else rows.to(DEV), rms=True, pending=pending)
        torch.testing.assert_close(out.cpu().double(), want_h if rows is None else want_h[rows.long()], **tol(dtype))
        if rows is None:
            torch.testing.assert_close(x.cpu().double(), want_x, rtol=1e-5, atol=1e-5)
            assert torch.equal(streams[n - 1].cpu(), results[n - 1])
            # and the same bits as the kernel that only sums
            x2 = results[n - 1].clone().to(DEV)
            K().stream_average(streams, x2, w.to(DEV), n)
            assert torch.equal(x2, x)


def run_attention(dtype, H, G, dk, dv, runs, window, cap, scale, q, k, v, talk, gate, ps=16, seed=0):
    """q [T, H*dk], k [Tk, G*dk], v [Tk, G*dv] per request given as lists (all keys of a request, the queries are its last
    tokens); through kv_write, attention_values and head_talk. Returns [T, H*dv] float64."""
    kern = K()
    kv_lens = [kv for _, kv in runs]
    n_pages = sum((n + ps - 1) // ps for n in kv_lens) + 3
    bt = random_block_tables(kv_lens, ps, n_pages, seed, DEV)
    k_pages = torch.full((n_pages, G * dk * ps), float("nan"), dtype=dtype, device=DEV)  # what a recycled page may hold
    v_pages = torch.full((n_pages, G * dv * ps), float("nan"), dtype=dtype, device=DEV)
    for s, n in enumerate(kv_lens):
        dest = torch.tensor([int(bt[s, p // ps]) * ps + p % ps for p in range(n)], dtype=torch.int32, device=DEV)
        kern.kv_write(k[s].to(dtype).to(DEV), v[s].to(dtype).to(DEV), k_pages, v_pages, dest, G, dk, ps, value_dim=dv)
    meta = make_meta(runs, DEV)
    qq = torch.cat(q).to(dtype).to(DEV)
    T = qq.shape[0]
    nv = G if talk is not None else 1
    o = torch.empty(T, H, nv, dv, dtype=torch.float32, device=DEV)
    slopes = Z.head_slopes(H).float().to(DEV)
    kern.attention_values(qq, o, k_pages, v_pages, meta, n_heads=H, n_kv_heads=G, head_dim=dk, value_dim=dv, all_value_heads=talk is not None,
                          page_size=ps, scale=scale, window=window, block_tables=bt, softcap=cap, slopes=slopes)
    a = torch.empty(T, H * dv, dtype=dtype, device=DEV)
    kern.head_talk(o, None if talk is None else talk.float().to(DEV), None if gate is None else gate.to(dtype).to(DEV), a, H, G, dv)
    return a.cpu().double()


def plain_attention(H, G, dk, dv, runs, window, cap, scale, q, k, v, talk, gate):
    outs, t0 = [], 0
    for s, (q_len, kv_len) in enumerate(runs):
        full_q = torch.zeros(kv_len, H, dk, dtype=torch.float64)
        full_q[kv_len - q_len:] = q[s].view(q_len, H, dk)
        w = Z.attention_weights(full_q, k[s].view(kv_len, G, dk), scale, cap, window)
        if talk is not None:
            w = Z.mix_heads(w, talk)
        o = Z.apply_weights(w, v[s].view(kv_len, G, dv))[kv_len - q_len:]
        if gate is not None:
            o = o * torch.sigmoid(gate[t0:t0 + q_len])[:, :, None]
        outs.append(o.reshape(q_len, H * dv))
        t0 += q_len
    return torch.cat(outs)


ATT_SHAPES = [  # H, G, dk, dv, window, cap
    (4, 2, 16, 8, 24, 10.0),
    (8, 2, 32, 16, 70, 15.0),
    (3, 3, 48, 32, None, None),
    (6, 1, 24, 40, 5, 3.0),
    (4, 4, 64, 64, 200, 20.0),
    (2, 1, 128, 16, 33, 50.0),
    (8, 8, 16, 64, 40, 10.0),   # more value heads than one wave of the matrix-core kernel takes
    (34, 2, 16, 16, 21, 10.0),  # more query heads per key/value head than a wave has columns
    (6, 6, 8, 408, 30, 10.0),   # more outputs a query head than a wave of the plain kernel holds (and no matrix-core kernel)
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", ATT_SHAPES)
@pytest.mark.parametrize("talking", [True, False])
def test_attention_prompts_portions_and_single_tokens(dtype, shape, talking):
    H, G, dk, dv, window, cap = shape
    g = torch.Generator().manual_seed(H * 100 + dk)
    runs = [(70, 70), (1, 130), (19, 83), (1, 1), (2, 2), (1, 17), (130, 261), (1, 48)]  # (queries, keys after the step)
    q = [as_bf16_numbers(Z.unit_rms(torch.randn(ql, H, dk, generator=g), 1e-6).reshape(ql, -1)) for ql, _ in runs]
    k = [as_bf16_numbers(Z.unit_rms(torch.randn(kl, G, dk, generator=g), 1e-6).reshape(kl, -1)) for _, kl in runs]
    v = [as_bf16_numbers(torch.randn(kl, G * dv, generator=g)) for _, kl in runs]
    T = sum(ql for ql, _ in runs)
    talk = as_bf16_numbers(torch.eye(H) + 0.5 * torch.randn(H, H, generator=g)) if talking else None
    gate = as_bf16_numbers(torch.randn(T, H, generator=g)) if talking else None
    scale = 4.0 / math.sqrt(dk)
    got = run_attention(dtype, H, G, dk, dv, runs, window, cap, scale, q, k, v, talk, gate, seed=dk)
    want = plain_attention(H, G, dk, dv, runs, window, cap, scale, q, k, v, talk, gate)
    torch.testing.assert_close(got, want, **tol(dtype, f32=3e-5, bf16=3e-2))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("single", [True, False])
@pytest.mark.parametrize("window,ps", [(24, 16), (16, 16), (33, 16), (64, 32), (1, 16), (129, 64)])
def test_a_key_just_inside_and_just_outside_the_window(dtype, single, window, ps):
    """One key carries a value far from all others and a score that stands out. At distance window - 1 the query's output
    is that value; at distance window it must not be seen at all. The last head's slope is small enough for the score to
    win at that distance; the query is the last token of a prompt, or a single token."""
    H, G, dk, dv = 2, 1, 16, 8
    n = window + 70
    g = torch.Generator().manual_seed(window)
    for dist, seen in ((window - 1, True), (window, False)):
        kk = as_bf16_numbers(Z.unit_rms(torch.randn(n, G, dk, generator=g), 1e-6) * 0.2)  # short keys: scores of a few units
        qq = as_bf16_numbers(Z.unit_rms(torch.randn(n, H, dk, generator=g), 1e-6))
        vv = as_bf16_numbers(torch.randn(n, G, dv, generator=g) * 0.1)
        j = n - 1 - dist
        kk[j, 0] = qq[n - 1, H - 1]  # the last head's query finds its own direction there
        vv[j, 0] = 100.0
        ql = 1 if single else 37
        runs = [(ql, n)]
        scale, cap = 2.0, 30.0  # the key of full length: cap(2 * 16) = 24, against keys with scores of a few units
        args = (H, G, dk, dv, runs, window, cap, scale, [qq[n - ql:].reshape(ql, -1)], [kk.reshape(n, -1)], [vv.reshape(n, -1)], None, None)
        got = run_attention(dtype, *args, ps=ps, seed=dist)
        want = plain_attention(*args)
        torch.testing.assert_close(got, want, **tol(dtype, f32=3e-5, bf16=3e-2))
        last = got[-1].view(H, dv)[H - 1]
        assert bool((last > 90).all()) == seen and (seen or bool((last.abs() < 5).all())), f"distance {dist} of window {window}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_key_among_hundreds_without_a_window(dtype):
    H, G, dk, dv = 4, 2, 32, 16
    n = 900
    g = torch.Generator().manual_seed(1)
    kk = as_bf16_numbers(Z.unit_rms(torch.randn(n, G, dk, generator=g), 1e-6) * 0.2)
    qq = as_bf16_numbers(Z.unit_rms(torch.randn(n, H, dk, generator=g), 1e-6))
    vv = as_bf16_numbers(torch.randn(n, G, dv, generator=g) * 0.1)
    kk[3, 1] = qq[n - 1, H - 1]  # slope of the last head: 2^-8, 3.5 at this distance
    vv[3, 1] = 50.0
    for ql in (1, 200):
        args = (H, G, dk, dv, [(ql, n)], None, 30.0, 1.0, [qq[n - ql:].reshape(ql, -1)], [kk.reshape(n, -1)], [vv.reshape(n, -1)], None, None)
        got = run_attention(dtype, *args)
        torch.testing.assert_close(got, plain_attention(*args), **tol(dtype, f32=3e-5, bf16=3e-2))
        assert bool((got[-1].view(H, dv)[H - 1] > 45).all())


# ------------------------------------------------------------------------------------------------ whole models
def model_folder(name, tmp, store):
    raw, seed = ZED[name]
    W = Z.random_weights(raw, seed)
    return raw, W, Z.write_folder(raw, W, os.path.join(str(tmp), name), store)


def row_error(got, want):
    """Difference of two rows of logits, mean taken off, relative to the spread of the wanted row."""
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / want.std(-1)).max().item()


LENGTHS = {"A": [70, 45, 100, 37, 64, 33], "B": [90, 130, 41, 200, 64, 17], "C": [40, 12, 30, 3], "D": [66, 21, 80, 5, 97]}


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_all_cuttings(name, dtype, tmp_path):
    """Whole prompts, the last 32 tokens one by one, portions down to two tokens, and twice mixed with other requests in a pool
    of exactly the peak need (pages and slots are used again), through ``bin/trace_run``."""
    from test_gpu_replay import read_step, run_trace

    raw, W, d = model_folder(name, tmp_path, torch.float32 if dtype == "float32" else torch.bfloat16)
    reqs = TR.random_requests(raw["vocab"], LENGTHS[name], 21)
    plain = {rid: Z.plain_logits(W, raw, torch.tensor(t)) for rid, t in reqs.items()}
    steps = TR.number(TR.trace_whole(reqs) + TR.trace_prefill_then_singles(reqs) + TR.trace_portions(reqs)
                      + TR.trace_mixed(reqs, seed=3) + TR.trace_mixed(reqs, seed=4, prefix="n"))
    out = run_trace(d, dtype, steps, TR.peak_tokens(steps))
    want = TR.expected_rows(steps, lambda rid: plain[rid[1:]])
    worst = 0.0
    for s in steps:
        k = s["step"]
        assert (k in want) == os.path.exists(os.path.join(out, f"{k}.f32"))
        if k in want:
            e = row_error(read_step(out, k, raw["vocab"]).double(), want[k])
            worst = max(worst, e)
            assert e < (1e-4 if dtype == "float32" else 6e-2), f"step {k} {s['entries'][0]['id']}: {e}"
    print(f"zederax {name} {dtype}: worst relative row error {worst:.3e}")


def _engine(d, dtype, **kw):
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import InferenceEngine

    cfg = InferenceEngineConfig(**{**dict(max_seqs=4, page_size=16, max_pages_per_seq=32, compute_dtype=dtype), **kw})
    return InferenceEngine.from_pretrained(d, cfg)


def check_greedy(W, raw, prompt, generated, margin):
    logits = Z.plain_logits(W, raw, torch.tensor(list(prompt) + list(generated)))
    clear = 0
    for i, tok in enumerate(generated):
        row = logits[len(prompt) - 1 + i]
        top = row.topk(2).values
        if float(top[0] - top[1]) > margin:
            clear += 1
            assert int(row.argmax()) == tok, f"generated token {i}"
    return clear


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(dtype, tmp_path):
    from levanter_amd.engine import Request

    raw, W, d = model_folder("A", tmp_path, torch.float32 if dtype == "float32" else torch.bfloat16)
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, raw["vocab"], (n,), generator=g).tolist() for n in (5, 17, 33, 1)]
    engine = _engine(d, dtype)
    res = engine.generate([Request(prompt_tokens=p, request_id=i, max_new_tokens=20) for i, p in enumerate(prompts)])
    assert [len(t) for t in res.tokens] == [20] * 4 and res.finish_reasons == ["length"] * 4
    margin = 1e-3 if dtype == "float32" else 0.3
    clear = sum(check_greedy(W, raw, p, out, margin) for p, out in zip(prompts, res.tokens))
    assert clear >= (76 if dtype == "float32" else 50)
    engine.cache.check_invariants()
    assert engine.cache.n_free_slots == 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_past_every_window_in_replayed_steps(dtype, tmp_path):
    """One prompt token, then 300 decoded ones: the windows (24, 37, 5 and none) pass over decoded tokens only, windowed
    groups give pages back on the way, and from the third step on the steps are replayed from a graph."""
    from levanter_amd.engine import Request

    raw, W, d = model_folder("A", tmp_path, torch.float32 if dtype == "float32" else torch.bfloat16)
    engine = _engine(d, dtype, max_pages=40)
    res = engine.generate([Request(prompt_tokens=[7], request_id=0, max_new_tokens=300)])
    out = res.tokens[0]
    assert len(out) == 300
    assert check_greedy(W, raw, [7], out, 1e-3 if dtype == "float32" else 0.3) >= (280 if dtype == "float32" else 150)
    # the first tokens of sequences of one, two and three tokens in one batch
    res = engine.generate([Request(prompt_tokens=p, request_id=i + 1, max_new_tokens=3) for i, p in enumerate(([5], [9, 4], [1, 2, 3]))])
    for p, o in zip(([5], [9, 4], [1, 2, 3]), res.tokens):
        check_greedy(W, raw, p, o, 1e-3 if dtype == "float32" else 0.3)
    engine.cache.check_invariants()


def test_the_command_line_generates_from_a_folder(tmp_path):
    """``python -m levanter_amd.main.sample_lm`` on a Zederax folder: greedy tokens are the plain implementation's."""
    import json
    import re
    import subprocess
    import sys

    raw, W, d = model_folder("C", tmp_path, torch.float32)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prompts = [[3, 14, 15, 9, 2], [6]]
    p = subprocess.run([sys.executable, "-m", "levanter_amd.main.sample_lm", "--hf_checkpoint", d, "--prompt_ids", json.dumps(prompts),
                        "--temperature", "0", "--max_new_tokens", "12", "--n_rounds", "1", "--engine.compute_dtype", "float32",
                        "--engine.max_seqs", "2", "--engine.max_pages_per_seq", "4"], capture_output=True, text=True, cwd=root, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    found = re.findall(r"round 0 sequence (\d+) \(12 tokens, length\): (\[.*\])", p.stdout)
    assert len(found) == 2
    for i, toks in found:
        check_greedy(W, raw, prompts[int(i)], json.loads(toks), 1e-3)
