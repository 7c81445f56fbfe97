"""Sequence-mixer models on the HIP path against the plain oracle (oracle/seqmix.py): every mechanism alone through its
own entry point of libumbrella_seq.so, then whole models through the runtime, the cache manager and the batch engine.

fp32 runs are the sharp ones (every comparison to ~1e-5); bf16 runs use inputs built so that a fault still shows."""
import json
import os
import subprocess
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))
F32_TOL = 2e-5
BF16_TOL = 4e-2


@pytest.fixture(scope="module")
def lib():
    import __graft_entry__ as ge
    from umbrella_amd import _lib
    if not os.path.exists(_lib.SEQ_LIB_PATH):
        ge.build_seq()
    return _lib.load_seq()


def dev(t, dtype=None):
    return t.to(device="cuda:0", dtype=dtype).contiguous()


# ------------------------------------------------------------------ linear
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,N,K", [(1, 16, 32), (3, 5, 7), (17, 40, 136), (33, 6, 24), (70, 130, 260), (16, 64, 1024)])
def test_linear_any_shape(lib, dtype, T, N, K):
    from umbrella_amd import _lib
    g = torch.Generator().manual_seed(T * 1000 + N + K)
    x, w, b = (torch.randn(s, generator=g).to(dtype) for s in ((T, K), (N, K), (N,)))
    want = x.double() @ w.double().T + b.double()
    out = torch.empty(T, N, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_seq_linear", out, dev(x), dev(w), dev(b), T, N, K, 0, _lib.seq_dtype_code(dtype))
    assert (out.cpu().double() - want).abs().max() < 1e-4 * K ** 0.5
    out_dt = torch.empty(T, N, dtype=dtype, device="cuda:0")
    _lib.seq_call("umb_seq_linear", out_dt, dev(x), dev(w), None, T, N, K, 1, _lib.seq_dtype_code(dtype))
    want_nb = x.double() @ w.double().T
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    assert (out_dt.cpu().double() - want_nb).abs().max() < tol * K ** 0.5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_silu_mul_epilogue(lib, dtype):
    from umbrella_amd import _lib
    T, Nh, K = 19, 24, 40
    g = torch.Generator().manual_seed(5)
    x, w = torch.randn(T, K, generator=g).to(dtype), (0.3 * torch.randn(2 * Nh, K, generator=g)).to(dtype)
    gate, up = x.double() @ w[:Nh].double().T, x.double() @ w[Nh:].double().T
    want = gate * torch.sigmoid(gate) * up
    out = torch.empty(T, Nh, dtype=dtype, device="cuda:0")
    _lib.seq_call("umb_seq_linear", out, dev(x), dev(w), None, T, 2 * Nh, K, 2, _lib.seq_dtype_code(dtype))
    rel = 1e-5 if dtype == torch.float32 else 2.0 ** -8          # one rounding of the result to the storage dtype
    assert ((out.cpu().double() - want).abs() <= rel * want.abs() + 1e-4).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,N,K", [(300, 200, 264), (257, 130, 72), (512, 256, 128)])
def test_linear_many_tokens_tiled_through_lds(lib, dtype, T, N, K):
    """prompts of >= 256 tokens take the 128 x 128 LDS-tiled kernel: ragged edges in all three dimensions, bias, the
    rounding epilogue and the gate/up epilogue"""
    from umbrella_amd import _lib
    g = torch.Generator().manual_seed(T + N + K)
    x, w, b = (torch.randn(s, generator=g).to(dtype) for s in ((T, K), (N, K), (N,)))
    code = _lib.seq_dtype_code(dtype)
    want = x.double() @ w.double().T + b.double()
    out = torch.empty(T, N, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_seq_linear", out, dev(x), dev(w), dev(b), T, N, K, 0, code)
    assert (out.cpu().double() - want).abs().max() < 1e-4 * K ** 0.5
    out_dt = torch.empty(T, N, dtype=dtype, device="cuda:0")
    _lib.seq_call("umb_seq_linear", out_dt, dev(x), dev(w), dev(b), T, N, K, 1, code)
    assert ((out_dt.cpu().double() - want).abs() <= 2.0 ** -8 * want.abs() + 1e-4 * K ** 0.5).all()
    w2 = (0.2 * torch.randn(2 * N, K, generator=g)).to(dtype)
    gate, up = x.double() @ w2[:N].double().T, x.double() @ w2[N:].double().T
    act = torch.empty(T, N, dtype=dtype, device="cuda:0")
    _lib.seq_call("umb_seq_linear", act, dev(x), dev(w2), None, T, 2 * N, K, 2, code)
    want_act = gate * torch.sigmoid(gate) * up
    assert ((act.cpu().double() - want_act).abs() <= 2.0 ** -8 * want_act.abs() + 1e-4 * K ** 0.5).all()
    # the same rows through the skinny kernel (<= 64 tokens): equal up to the order of the fp32 sums
    few = torch.empty(40, N, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_seq_linear", few, dev(x[100:140]), dev(w), dev(b), 40, N, K, 0, code)
    assert (few - out[100:140]).abs().max() < 1e-4 * K ** 0.5


def test_linear_rows_do_not_depend_on_the_batch(lib):
    """a row's result is bit-identical whether it is computed alone, in a tile of 16 or among 70 rows"""
    from umbrella_amd import _lib
    g = torch.Generator().manual_seed(1)
    x, w = dev(torch.randn(70, 200, generator=g), torch.bfloat16), dev(torch.randn(48, 200, generator=g), torch.bfloat16)
    full = torch.empty(70, 48, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_seq_linear", full, x, w, None, 70, 48, 200, 0, _lib.BF16)
    for lo, n in ((0, 1), (5, 11), (40, 30)):
        part = torch.empty(n, 48, dtype=torch.float32, device="cuda:0")
        _lib.seq_call("umb_seq_linear", part, x[lo:lo + n].contiguous(), w, None, n, 48, 200, 0, _lib.BF16)
        assert torch.equal(part, full[lo:lo + n])


# ------------------------------------------------------------------ norms
@pytest.mark.parametrize("groups,W", [(1, 40), (4, 64), (3, 201), (2, 1280), (1, 1100)])
def test_group_norm_and_residual_seam(lib, groups, W):
    from oracle import seqmix as O
    from umbrella_amd import _lib
    T, eps = 5, 1e-5
    g = torch.Generator().manual_seed(groups + W)
    x, y = torch.randn(T, W, generator=g) * 3, torch.randn(T, W, generator=g) * 50
    w1, w2 = 1 + 0.2 * torch.randn(W, generator=g), 1 + 0.2 * torch.randn(W, generator=g)
    out = torch.empty(T, W, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_seq_group_norm", out, None, dev(x), None, dev(w1), T, W, groups, eps, _lib.F32)
    assert (out.cpu().double() - O.group_rms_norm(x.double(), w1.double(), groups, eps)).abs().max() < 1e-5
    rows = torch.tensor([3, 0], dtype=torch.int32, device="cuda:0")            # gathered rows
    _lib.seq_call("umb_seq_group_norm", out, None, dev(x), rows, dev(w1), 2, W, groups, eps, _lib.F32)
    assert (out[:2].cpu().double() - O.group_rms_norm(x[[3, 0]].double(), w1.double(), groups, eps)).abs().max() < 1e-5
    xd, h = dev(x), torch.empty(T, W, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_seq_resid_norm", xd, h, dev(y), dev(w1), dev(w2), T, W, groups, eps, _lib.F32)
    x_new = x.double() + O.group_rms_norm(y.double(), w1.double(), groups, eps)
    assert (xd.cpu().double() - x_new).abs().max() < 1e-5
    assert (h.cpu().double() - O.group_rms_norm(x_new, w2.double(), groups, eps)).abs().max() < 1e-5


# ------------------------------------------------------------------ gated linear attention, alone
def _gla_weights(width, H, D, E, rank, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g)  # noqa: E731
    return dict(wq=r(H * D, width) / width ** 0.5, wk=r(H * D, width) / width ** 0.5, wv=r(H * E, width) / width ** 0.5,
                wg=r(H * E, width) / width ** 0.5, wo=r(width, H * E) / (H * E) ** 0.5, w_norm=1 + 0.1 * r(E),
                wa1=r(rank, width) / width ** 0.5, wa2=r(H * D, rank), ba2=2.0 + r(H * D))


def _run_gla(X, w, H, D, E, tau, eps, state, slot, pos0, splits):
    """the library's decay -> scan -> gate on the rows of X, cut into consecutive parts of the given sizes"""
    from umbrella_amd import _lib
    width = X.shape[1]
    proj_w = dev(torch.cat([w["wq"], w["wk"], w["wv"], w["wg"], w["wa1"]]))
    ld, rank = proj_w.shape[0], w["wa1"].shape[0]
    outs, at = [], 0
    for n in splits:
        x = dev(X[at:at + n].float())
        proj = torch.empty(n, ld, dtype=torch.float32, device="cuda:0")
        _lib.seq_call("umb_seq_linear", proj, x, proj_w, None, n, ld, width, 0, _lib.F32)
        alpha = torch.empty(n, H * D, dtype=torch.float32, device="cuda:0")
        _lib.seq_call("umb_gla_decay", alpha, proj, ld, 2 * H * D + 2 * H * E, dev(w["wa2"]), dev(w["ba2"]), n, H * D, rank,
                      float(tau), _lib.F32)
        o = torch.empty(n, H * E, dtype=torch.float32, device="cuda:0")
        meta = torch.tensor([slot, 0, pos0 + at, n], dtype=torch.int32, device="cuda:0")
        _lib.seq_call("umb_gla_scan", o, state, proj, ld, alpha, meta[0:1], meta[1:2], meta[2:3], meta[3:4], 1, H, D, E,
                      float(D) ** -0.5)
        mix = torch.empty(n, H * E, dtype=torch.float32, device="cuda:0")
        _lib.seq_call("umb_gla_gate", mix, o, proj, ld, 2 * H * D + H * E, dev(w["w_norm"]), n, H, E, eps, _lib.F32)
        y = torch.empty(n, width, dtype=torch.float32, device="cuda:0")
        _lib.seq_call("umb_seq_linear", y, mix, dev(w["wo"]), None, n, width, H * E, 0, _lib.F32)
        outs.append(y)
        at += n
    return torch.cat(outs)


@pytest.mark.parametrize("H,D,E,rank,tau", [(2, 16, 8, 4, 8.0), (3, 24, 20, 5, 1.0), (1, 130, 70, 16, 32.0), (2, 7, 3, 1, 2.5), (1, 256, 18, 3, 4.0),
                                              (2, 64, 32, 8, 4.0), (1, 128, 16, 4, 16.0)])
def test_gla_alone_prefill_and_token_by_token(lib, H, D, E, rank, tau):
    from oracle import seqmix as O
    width, n, eps = 40, 37, 1e-5
    w = _gla_weights(width, H, D, E, rank, seed=H * 100 + D)
    X = torch.randn(n, width, generator=torch.Generator().manual_seed(3))
    want, S_want = O.gated_linear_attention(X.double(), *(w[k].double() for k in ("wq", "wk", "wv", "wg", "wo", "w_norm", "wa1",
                                                                                  "wa2", "ba2")), H=H, D=D, E=E, tau=tau, eps=eps)
    # the slot holds garbage from an earlier sequence: a sequence that starts at position 0 must not see it
    state = torch.full((3, H, D, E), float("nan"), dtype=torch.float32, device="cuda:0")
    whole = _run_gla(X, w, H, D, E, tau, eps, state, slot=1, pos0=0, splits=[n])
    assert (whole.cpu().double() - want).abs().max() < 2e-4
    assert (state[1].cpu().double() - S_want).abs().max() < 2e-4
    assert torch.isnan(state[0]).all() and torch.isnan(state[2]).all()           # other slots untouched
    state2 = torch.full((3, H, D, E), float("nan"), dtype=torch.float32, device="cuda:0")
    steps = _run_gla(X, w, H, D, E, tau, eps, state2, slot=2, pos0=0, splits=[1] * n)
    assert (steps - whole).abs().max() < 1e-5
    state3 = torch.full((3, H, D, E), float("nan"), dtype=torch.float32, device="cuda:0")
    parts = _run_gla(X, w, H, D, E, tau, eps, state3, slot=0, pos0=0, splits=[2, 9, 1, 20, 5])
    assert (parts - whole).abs().max() < 1e-5


def test_gla_far_token_survives_long_decoding(lib):
    """one early token writes a large value through a channel that barely decays; 300 tokens later the state still
    carries it, through single-token steps, exactly as the recurrence says"""
    from oracle import seqmix as O
    H, D, E, rank, tau, width, n, eps = 1, 16, 8, 2, 64.0, 24, 300, 1e-5
    w = _gla_weights(width, H, D, E, rank, seed=9)
    w["ba2"] = torch.full((H * D,), 6.0)                       # alpha ~ 1 - 4e-5 per token
    X = 0.05 * torch.randn(n, width, generator=torch.Generator().manual_seed(4))
    X[3] *= 200.0                                              # the token to remember
    want, _ = O.gated_linear_attention(X.double(), *(w[k].double() for k in ("wq", "wk", "wv", "wg", "wo", "w_norm", "wa1", "wa2",
                                                                             "ba2")), H=H, D=D, E=E, tau=tau, eps=eps)
    state = torch.zeros(1, H, D, E, dtype=torch.float32, device="cuda:0")
    got = _run_gla(X, w, H, D, E, tau, eps, state, slot=0, pos0=0, splits=[8] + [1] * (n - 8))
    scale = float(want[50:].abs().max())                       # the quiet tail, far behind the loud token
    assert (got.cpu().double() - want)[50:].abs().max() < 1e-3 * scale
    assert (got.cpu().double() - want).abs().max() < 1e-4 * float(want.abs().max())
    forgot = X.clone()
    forgot[3] = 0
    lost, _ = O.gated_linear_attention(forgot.double(), *(w[k].double() for k in ("wq", "wk", "wv", "wg", "wo", "w_norm", "wa1",
                                                                                  "wa2", "ba2")), H=H, D=D, E=E, tau=tau, eps=eps)
    assert (want[-1] - lost[-1]).abs().max() > 0.2 * scale     # a lost state is 200 times the tolerance


# ------------------------------------------------------------------ pooled-window attention, alone
def _attn_weights(width, H, G, D, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g)  # noqa: E731
    return dict(wq=r(H * D, width) / width ** 0.5, bq=0.3 * r(H * D), wk=r(G * D, width) / width ** 0.5, bk=0.3 * r(G * D),
                wg=r(H, width) / width ** 0.5, wo=r(width, H * D) / (H * D) ** 0.5, bo=0.1 * r(width), pb=0.5 * r(H))


def _run_attn(X, w, H, G, D, window, pool, rot_dims, base, scale, eps, dtype, page, splits, seq="s", cache=None, tiled=False):
    """the library's prep -> pool -> attend on the rows of X through a paged cache, cut into consecutive steps"""
    from umbrella_amd import _lib
    from umbrella_amd.attn.cache import PagedSeqCache
    width, code = X.shape[1], _lib.seq_dtype_code(dtype)
    if cache is None:
        cache = PagedSeqCache([(G, D, pool)], [], max_tokens=X.shape[0] + 2 * page, max_seqs=2, device="cuda:0", dtype=dtype,
                              page=page)
    cache.open(seq)
    kv = cache.struct(0)
    proj_w = dev(torch.cat([w["wq"], w["wk"], w["wg"]]), dtype)
    proj_b = dev(torch.cat([w["bq"], w["bk"], torch.zeros(H)]), dtype)
    freq = dev(base ** (-2 * torch.arange(rot_dims // 2, dtype=torch.float32) / rot_dims)) if rot_dims else None
    ld, outs, at = proj_w.shape[0], [], 0
    for n in splits:
        p0, slot = cache.extend(seq, n), cache.slot(seq)
        x = dev(X[at:at + n], dtype)
        proj = torch.empty(n, ld, dtype=torch.float32, device="cuda:0")
        _lib.seq_call("umb_seq_linear", proj, x, proj_w, proj_b, n, ld, width, 0, code)
        pos = torch.arange(p0, p0 + n, dtype=torch.int32, device="cuda:0")
        slots = torch.full((n,), slot, dtype=torch.int32, device="cuda:0")
        meta = torch.tensor([slot, p0, n], dtype=torch.int32, device="cuda:0")
        q = torch.empty(n, H * D, dtype=torch.float32, device="cuda:0")
        _lib.seq_call("umb_pwa_prep", q, kv, proj, ld, pos, slots, freq, n, H, G, D, rot_dims, eps, code)
        _lib.seq_call("umb_pwa_pool", kv, meta[0:1], meta[1:2], meta[2:3], 1, n, G, D, pool, code)
        mix = torch.empty(n, H * D, dtype=dtype, device="cuda:0")
        if tiled and n >= 16:                # as the model does: stretches of a sequence go to the matrix-pipe kernel
            one = torch.tensor([0], dtype=torch.int32, device="cuda:0")
            _lib.seq_call("umb_pwa_attend_tiled", mix, q, kv, proj, ld, H * D + G * D, dev(w["pb"], dtype), meta[0:1], one,
                          meta[1:2], meta[2:3], 1, n, H, G, D, window, pool, float(scale), code)
        else:
            _lib.seq_call("umb_pwa_attend", mix, q, kv, proj, ld, H * D + G * D, dev(w["pb"], dtype), pos, slots, n, H, G, D,
                          window, pool, float(scale), code)
        y = torch.empty(n, width, dtype=torch.float32, device="cuda:0")
        _lib.seq_call("umb_seq_linear", y, mix, dev(w["wo"], dtype), dev(w["bo"], dtype), n, width, H * D, 0, code)
        outs.append(y)
        at += n
    return torch.cat(outs), cache


def _attn_oracle(X, w, dtype, **kw):
    from oracle import seqmix as O
    r = (lambda t: t.to(dtype).double()) if dtype != torch.float32 else (lambda t: t.float().double())
    ws = {k: r(v) for k, v in w.items()}
    return O.pooled_window_attention(r(X), ws["wq"], ws["bq"], ws["wk"], ws["bk"], ws["wg"], ws["wo"], ws["bo"], ws["pb"],
                                     cache_round=None if dtype == torch.float32 else r, **kw)


ATTN_CASES = [  # H, G, D, window, pool, rot_dims, page
    (4, 2, 16, 6, 3, 16, 4), (2, 2, 24, 5, 2, 8, 64), (3, 1, 10, 1, 1, 4, 3), (2, 1, 32, 9, 7, 32, 5), (6, 3, 8, 4, 11, 0, 4),
    (1, 1, 70, 3, 2, 6, 7), (8, 1, 16, 7, 2, 16, 8), (9, 3, 8, 3, 3, 8, 4)]


@pytest.mark.parametrize("H,G,D,window,pool,rot_dims,page", ATTN_CASES)
def test_attention_alone_every_position(lib, H, G, D, window, pool, rot_dims, page):
    """every position of a 45-token sequence (so: every phase of window, block and page) in fp32, whole and cut up"""
    width, n, eps, base = 40, 45, 1e-5, 100.0
    w = _attn_weights(width, H, G, D, seed=H * 10 + D)
    X = torch.randn(n, width, generator=torch.Generator().manual_seed(8))
    kw = dict(H=H, G=G, D=D, window=window, pool=pool, rot_dims=rot_dims, base=base, scale=0.37, eps=eps)
    want = _attn_oracle(X, w, torch.float32, **kw)
    whole, _ = _run_attn(X, w, dtype=torch.float32, page=page, splits=[n], **kw)
    assert (whole.cpu().double() - want).abs().max() < 1e-4
    steps, _ = _run_attn(X, w, dtype=torch.float32, page=page, splits=[1] * n, **kw)
    assert (steps - whole).abs().max() < 1e-5
    parts, _ = _run_attn(X, w, dtype=torch.float32, page=page, splits=[2, 13, 1, 1, 20, 3, 5], **kw)
    assert (parts - whole).abs().max() < 1e-5


def test_attention_many_rounds_of_keys(lib):
    """a window and a pooled history that each span several 64-key rounds (and 32-key steps), in prompts and in decoding"""
    H, G, D, window, pool, page, width, n, eps = 2, 1, 32, 100, 2, 16, 24, 300, 1e-5
    w = _attn_weights(width, H, G, D, seed=77)
    X = torch.randn(n, width, generator=torch.Generator().manual_seed(5))
    kw = dict(H=H, G=G, D=D, window=window, pool=pool, rot_dims=16, base=1000.0, scale=0.1, eps=eps)
    want = _attn_oracle(X, w, torch.float32, **kw)
    whole, _ = _run_attn(X, w, dtype=torch.float32, page=page, splits=[n], **kw)
    scale = float(want.abs().max())
    assert (whole.cpu().double() - want).abs().max() < 2e-5 * scale
    steps, _ = _run_attn(X, w, dtype=torch.float32, page=page, splits=[250] + [1] * 50, **kw)
    assert (steps - whole).abs().max() < 2e-5 * scale
    want16 = _attn_oracle(X, w, torch.bfloat16, **kw)
    tiled, _ = _run_attn(X, w, dtype=torch.bfloat16, page=page, splits=[140, 160], tiled=True, **kw)
    assert (tiled.cpu().double() - want16).abs().max() < 1.2e-2 * scale


def _standout(n, width, H, G, D, loud):
    """weights and inputs under which every key is (almost) invisible except the tokens in `loud`, each of which has weight
    1/2 for every later query: constant projections, a strongly negative score bias, keys that point along the query for
    loud tokens and against it for all others"""
    w = dict(wq=torch.zeros(H * D, width), bq=torch.ones(H * D), wk=torch.zeros(G * D, width), bk=torch.full((G * D,), 1e-3),
             wg=torch.zeros(H, width), wo=torch.zeros(width, H * D), bo=torch.zeros(width), pb=torch.full((H,), -12.0))
    w["wk"][:, 0] = 1.0                                # key = x[0] * ones: +ones (loud) or -ones (quiet) after unit RMS
    for c in range(min(width, H * D)):
        w["wo"][c, c] = 1.0
    X = torch.zeros(n, width)
    X[:, 0] = -1.0
    X[loud, 0] = 1.0
    return w, X


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_window_and_pool_edges_with_standout_keys(lib, dtype):
    """The four tokens of one block carry all the weight (score 0 -> weight 1/2 each, value ~1, gate 1/2: each adds 1/4 to
    the output; every other key adds ~1e-11).  So the output COUNTS what a query sees: the loud tokens still in its window,
    nothing for those that have left it, and from exactly the position where the block lies wholly behind the window one
    pooled key.  An edge that is one position off changes a count.  Checked in prompts and in decoding, pages < block."""
    H, G, D, window, pool, page, width, n, eps = 2, 1, 8, 5, 4, 3, 16, 40, 1e-6
    loud = [8, 9, 10, 11]                              # block 2
    w, X = _standout(n, width, H, G, D, loud)
    kw = dict(H=H, G=G, D=D, window=window, pool=pool, rot_dims=0, base=10.0, scale=1.5, eps=eps)
    want = _attn_oracle(X, w, dtype, **kw)
    count = (want[:, 0] / 0.25).round().int().tolist()
    #        i = 7  8  9 10 11 12 13 14 15 | 16: the block is seen (11 <= 16 - 5), its tokens are out of the window
    assert count[7:17] == [0, 1, 2, 3, 4, 4, 3, 2, 1, 1] and count[17:] == [1] * (n - 17)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for splits in ([n], [12] + [1] * (n - 12), [16] + [1] * (n - 16), [15] + [1] * (n - 15), [2] * (n // 2)):
        got, _ = _run_attn(X, w, dtype=dtype, page=page, splits=splits, **kw)
        assert (got.cpu().double() - want).abs().max() < tol, splits


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("H,G,D,window,pool,rot_dims,page", [(4, 2, 32, 6, 3, 32, 4), (8, 2, 64, 9, 7, 16, 5), (3, 3, 32, 1, 1, 8, 3),
                                                             (2, 1, 96, 20, 4, 0, 64), (2, 1, 128, 12, 5, 64, 8),
                                                             (1, 1, 256, 7, 2, 256, 16)])
def test_attention_on_the_matrix_pipe(lib, dtype, H, G, D, window, pool, rot_dims, page):
    """prompt stretches of >= 16 tokens through the MFMA kernel (every phase of window, block, page and 16-query tile),
    against the oracle and against the vector-pipe kernel: the two must agree to the rounding of their 16-bit outputs"""
    width, n, eps, base = 40, 70, 1e-5, 100.0
    w = _attn_weights(width, H, G, D, seed=H + D)
    X = torch.randn(n, width, generator=torch.Generator().manual_seed(11))
    kw = dict(H=H, G=G, D=D, window=window, pool=pool, rot_dims=rot_dims, base=base, scale=0.21, eps=eps)
    want = _attn_oracle(X, w, dtype, **kw)
    plain, _ = _run_attn(X, w, dtype=dtype, page=page, splits=[n], **kw)
    # the mixer output is rounded to the storage dtype before the output projection: errors scale with the outputs
    tol = (1.2e-2 if dtype == torch.bfloat16 else 2e-3) * max(1.0, float(want.abs().max()))
    assert (plain.cpu().double() - want).abs().max() < tol
    for splits in ([n], [33, 37], [16, 16, 16, 16, 6], [20] + [1] * 50, [17, 1, 1, 18, 33]):
        got, _ = _run_attn(X, w, dtype=dtype, page=page, splits=splits, tiled=True, **kw)
        assert (got.cpu().double() - want).abs().max() < tol, splits
        assert (got - plain).abs().max() < tol / 2, splits


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_matrix_pipe_window_and_pool_edges_with_standout_keys(lib, dtype):
    """the counting test of the vector-pipe kernel, on the MFMA kernel: tiles of 16 queries that straddle every edge"""
    H, G, D, window, pool, page, width, n, eps = 2, 1, 32, 5, 4, 3, 16, 48, 1e-6
    loud = [8, 9, 10, 11]
    w, X = _standout(n, width, H, G, D, loud)
    kw = dict(H=H, G=G, D=D, window=window, pool=pool, rot_dims=0, base=10.0, scale=12.0 / D, eps=eps)
    want = _attn_oracle(X, w, dtype, **kw)
    count = (want[:, 0] / 0.25).round().int().tolist()
    assert count[7:17] == [0, 1, 2, 3, 4, 4, 3, 2, 1, 1] and count[17:] == [1] * (n - 17)
    for splits in ([n], [16, 32], [24, 24], [17, 31]):
        got, _ = _run_attn(X, w, dtype=dtype, page=page, splits=splits, tiled=True, **kw)
        assert (got.cpu().double() - want).abs().max() < 2e-2, splits


def test_attention_pages_are_reused_without_leaking(lib):
    """sequence B runs in the pages and the slot that sequence A has just given back: same result as in a fresh cache"""
    H, G, D, window, pool, page, width, eps = 2, 2, 8, 4, 3, 4, 16, 1e-5
    w = _attn_weights(width, H, G, D, seed=2)
    kw = dict(H=H, G=G, D=D, window=window, pool=pool, rot_dims=8, base=50.0, scale=0.4, eps=eps)
    A = 5 * torch.randn(30, width, generator=torch.Generator().manual_seed(1))
    Bx = torch.randn(22, width, generator=torch.Generator().manual_seed(2))
    fresh, _ = _run_attn(Bx, w, dtype=torch.bfloat16, page=page, splits=[10] + [1] * 12, **kw)
    _, cache = _run_attn(A, w, dtype=torch.bfloat16, page=page, splits=[30], seq="a", **kw)
    pages_a = list(cache.seqs["a"]["pages"])
    cache.close("a")
    again, cache = _run_attn(Bx, w, dtype=torch.bfloat16, page=page, splits=[10] + [1] * 12, seq="b", cache=cache, **kw)
    assert set(cache.seqs["b"]["pages"]) <= set(pages_a) and cache.slot("b") == 0
    assert torch.equal(again, fresh)


# ------------------------------------------------------------------ whole models through the runtime
def _oracle_logits(cfgd, sd, toks, dtype):
    from oracle import seqmix as O
    r = None if dtype == torch.float32 else (lambda t: t.to(dtype).double())
    return O.gitopel_forward(cfgd, sd, toks, cache_round=r)


@pytest.mark.parametrize("name", ["mixed", "gla_first", "wide_pool"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_prefill_decode_portions_against_oracle(lib, name, dtype):
    from seqmix_helpers import CONFIGS, build, rel_err, tokens
    cfgd = CONFIGS[name]
    m, sd = build(cfgd, dtype, seed=11, page=4)
    n = 41
    toks = tokens(n, cfgd["vocab"], seed=5)
    want = _oracle_logits(cfgd, sd, toks, dtype)
    tol = F32_TOL if dtype == torch.float32 else BF16_TOL
    m.open("w")
    whole = m.forward_batch([("w", toks)], want=[list(range(n))]).clone()
    assert rel_err(whole, want) < tol
    same = F32_TOL if dtype == torch.float32 else 2e-2          # the model against itself under another schedule
    for sid, splits in (("d", [1] * n), ("p", [2, 2, 7, 1, 16, 3, 10]), ("q", [30] + [1] * 11)):
        m.open(sid)
        rows, at = [], 0
        for k in splits:
            rows.append(m.forward_batch([(sid, toks[at:at + k])], want=[list(range(k))]).clone())
            at += k
        got = torch.cat(rows)
        assert rel_err(got, want) < tol, (sid, "against the oracle")
        assert rel_err(got, whole) < same, (sid, "against the whole prompt")
        m.close(sid)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_unequal_batch_equals_each_alone(lib, dtype):
    """three requests of different lengths prefilled in one step and decoded together, the shortest ending first, against
    each of them alone; then a new request in the slot and pages the shortest one gave back"""
    from seqmix_helpers import CONFIGS, build, rel_err, tokens
    cfgd = CONFIGS["mixed"]
    m, _ = build(cfgd, dtype, seed=3, page=4, batch=3)
    V = cfgd["vocab"]
    seqs = {"a": tokens(33, V, 1), "b": tokens(9, V, 2), "c": tokens(21, V, 3)}
    pre = {"a": 20, "b": 1, "c": 13}
    alone = {}
    for k, t in seqs.items():
        m.open(k)
        alone[k] = m.forward_batch([(k, t)], want=[list(range(len(t)))]).clone()
        m.close(k)
    got = {k: [] for k in seqs}
    for k in seqs:
        m.open(k)
    out = m.forward_batch([(k, seqs[k][:pre[k]]) for k in seqs], want=[list(range(pre[k])) for k in seqs]).clone()
    at = 0
    for k in seqs:
        got[k].append(out[at:at + pre[k]])
        at += pre[k]
    done = dict(pre)
    late = None
    while any(done[k] < len(seqs[k]) for k in seqs):
        live = [k for k in seqs if done[k] < len(seqs[k])]
        out = m.forward_batch([(k, [seqs[k][done[k]]]) for k in live], want=[[0]] * len(live)).clone()
        for i, k in enumerate(live):
            got[k].append(out[i:i + 1])
            done[k] += 1
            if done[k] == len(seqs[k]):
                m.close(k)
                if k == "b":                            # its slot and pages go to a newcomer while a and c go on
                    late = tokens(15, V, 4)
                    seqs["z"], done["z"], got["z"] = late, 0, []
                    m.open("z")
                    assert m.kv_cache.slot("z") == 1
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    m.open("z0")
    alone["z"] = m.forward_batch([("z0", late)], want=[list(range(len(late)))]).clone()
    for k in seqs:
        assert rel_err(torch.cat(got[k]), alone[k]) < tol, k


def test_model_long_decoding_and_first_tokens(lib):
    """200 single-token steps over pages of 8 with a window of 6 and blocks of 3 (so every alignment of window, block and
    page occurs many times), against the oracle; and the first positions, where window and blocks are still empty"""
    from seqmix_helpers import attn_layer, config, gla_layer, build, rel_err, tokens
    cfgd = config([attn_layer(heads=2, kv_heads=1, dim=8, window=6, pool=3, ff=16), gla_layer(heads=1, dim=8, vdim=8, tau=4.0)],
                  vocab=40, width=24)
    m, sd = build(cfgd, torch.float32, seed=7, page=8, max_length=256)
    toks = tokens(200, 40, seed=6)
    want = _oracle_logits(cfgd, sd, toks, torch.float32)
    m.open("s")
    rows = [m.forward_batch([("s", [t])], want=[[0]]).clone() for t in toks]
    got = torch.cat(rows)
    assert rel_err(got[:12], want[:12]) < F32_TOL
    assert rel_err(got, want) < 5e-5
    assert len(m.kv_cache.seqs["s"]["pages"]) == 25


def test_decode_steps_replayed_as_graphs_equal_eager_launches(lib):
    """decode steps of a batch size are captured once and replayed; between replays the cache manager hands out pages, a
    request ends, a prompt of another request is prefilled eagerly: every replay must give what eager launches give"""
    from seqmix_helpers import CONFIGS, build, tokens
    cfgd = CONFIGS["mixed"]
    V = cfgd["vocab"]
    outs = []
    for graph in (True, False):
        from umbrella_amd.models import gitopel
        cfg = gitopel.config_from_dict(cfgd)
        sd = gitopel.synth_state(cfg, seed=13, rank=6)
        m = gitopel.Gitopel("tiny", batch_size=4, max_length=128, max_tokens=512, device="cuda:0", dtype=torch.bfloat16,
                            state_dict=sd, config=cfg, page_size=4, hip_graph=graph)
        m.alloc()
        got = []
        for k in "abc":
            m.open(k)
        got.append(m.forward_batch([("a", tokens(9, V, 1)), ("b", tokens(3, V, 2)), ("c", tokens(17, V, 3))]).clone())
        for i in range(10):                                    # three sequences: first step eager, second captured, then replays
            got.append(m.forward_batch([(k, [(7 * i + j) % V]) for j, k in enumerate("abc")]).clone())
        m.close("b")
        m.open("d")
        got.append(m.forward_batch([("d", tokens(6, V, 4))]).clone())            # eager work between replays
        for i in range(6):                                     # the same batch size again, another sequence in the slot
            got.append(m.forward_batch([(k, [(5 * i + j) % V]) for j, k in enumerate("adc")]).clone())
        for i in range(3):                                     # another batch size: its own graph
            got.append(m.forward_batch([(k, [(3 * i + j) % V]) for j, k in enumerate("ad")], want=[[0], []]).clone())
        assert (len(m._graphs) >= 2 and all(e["graph"] is not None for e in m._graphs.values())) == graph
        outs.append(got)
    for a, b in zip(*outs):
        assert torch.equal(a, b)


def test_cache_runs_out_loudly_and_recovers(lib):
    from seqmix_helpers import CONFIGS, build, tokens
    m, _ = build(CONFIGS["mixed"], torch.bfloat16, page=4, batch=2, max_tokens=16, max_length=64)
    m.open("a")
    m.forward_batch([("a", tokens(16, 96, 1))])
    m.open("b")
    m.forward_batch([("b", tokens(4, 96, 2))])
    with pytest.raises(RuntimeError):
        m.forward_batch([("b", tokens(8, 96, 3))])
    with pytest.raises(RuntimeError):
        m.open("c")
    m.close("a")
    m.forward_batch([("b", tokens(8, 96, 3))])


# ------------------------------------------------------------------ engine, scheduler, entry points
def _engine(cfgd, dtype, sd=None, **kw):
    from seqmix_helpers import build
    from umbrella_amd.speculation.auto_engine import AutoEngine
    from umbrella_amd.speculation.speculation_utils import IdTokenizer
    m, sd = build(cfgd, dtype, seed=21, page=4, batch=kw.pop("batch", 3), max_length=96, max_tokens=kw.pop("max_tokens", 512), sd=sd)
    e = AutoEngine.from_config("cuda:0", engine="batch", model="tiny", dtype=dtype, target_model_obj=m, tokenizer=IdTokenizer(), **kw)
    e.initialize()
    return e, sd


def _oracle_greedy(cfgd, sd, prompt, n):
    from oracle import seqmix as O
    toks, margins = list(prompt), []
    for _ in range(n):
        row = O.gitopel_forward(cfgd, sd, toks)[-1]
        top = torch.topk(row, 2).values
        margins.append(float(top[0] - top[1]))
        toks.append(int(row.argmax()))
    return toks[len(prompt):], margins


def test_engine_greedy_generation_matches_oracle(lib):
    """five queued requests through the scheduler (three slots: two batches), greedy, fp32: the oracle's tokens"""
    from seqmix_helpers import CONFIGS, tokens
    cfgd = CONFIGS["gla_first"]
    e, sd = _engine(cfgd, torch.float32)
    prompts = [tokens(n, cfgd["vocab"], seed=n) for n in (7, 1, 12, 3, 9)]
    outs = e.generate_batch(prompts, max_new_tokens=10)
    for p, got in zip(prompts, outs):
        want, margins = _oracle_greedy(cfgd, sd, p, 10)
        k = next((i for i, (a, b) in enumerate(zip(got, want)) if a != b), None)
        assert k is None or margins[k] < 1e-4, (got, want, margins)
    assert not e.target_model.kv_cache.seqs and len(e.target_model.kv_cache.free_slots) == 3
    # the conversation face of the same engine: prefill -> decode steps (verify) -> the same tokens
    assert e._prefill(torch.tensor([prompts[0]]))
    chat = []
    for _ in range(10):
        e.build_tree()
        e.verify()
        chat.append(e._chat.generated[-1])
    assert chat == outs[0]
    api = e.generate(input_ids=prompts[2], max_new_tokens=10)
    assert api["generated_tokens"] == outs[2]


def test_engine_sampling_is_seeded_and_in_range(lib):
    from seqmix_helpers import CONFIGS, tokens
    cfgd = CONFIGS["mixed"]
    e, _ = _engine(cfgd, torch.bfloat16, temperature=0.8, topk=8, topp=0.9, repetition_penalty=1.2, seed=5)
    prompts = [tokens(6, cfgd["vocab"], seed=1), tokens(11, cfgd["vocab"], seed=2)]
    a = e.generate_batch(prompts, max_new_tokens=12)
    e.reset()
    e.manual_seed(5)
    e.step_count.zero_()
    b = e.generate_batch(prompts, max_new_tokens=12)
    assert a == b and all(0 <= t < cfgd["vocab"] for o in a for t in o) and all(len(o) == 12 for o in a)


def test_trace_replay_command(lib, tmp_path):
    """bin/trace_run on a checkpoint directory: a mixed batch prefilled, decoded together, one request ending early"""
    from safetensors.torch import save_file
    from seqmix_helpers import CONFIGS, checkpoint, rel_err, tokens
    cfgd = CONFIGS["wide_pool"]
    _, sd = checkpoint(cfgd, seed=4)
    sd = {k: v.to(torch.bfloat16) for k, v in sd.items()}
    mdir, out = tmp_path / "model", tmp_path / "out"
    mdir.mkdir()
    save_file({k: v.contiguous() for k, v in sd.items()}, str(mdir / "model.safetensors"))
    (mdir / "config.json").write_text(json.dumps(cfgd))
    V = cfgd["vocab"]
    a, b = tokens(26, V, 1), tokens(8, V, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:20], "want": [0, 19]}, {"id": "b", "tokens": b[:5], "want": [4]}],
              "end": []}]
    for i in range(6):
        ent = [{"id": "a", "tokens": [a[20 + i]], "want": [0]}]
        if 5 + i < len(b):
            ent.append({"id": "b", "tokens": [b[5 + i]], "want": [] if i == 1 else [0]})
        steps.append({"step": i + 1, "entries": ent, "end": (["b"] if 5 + i == len(b) - 1 else []) + (["a"] if i == 5 else [])})
    for dt, tol in (("float32", F32_TOL), ("bfloat16", BF16_TOL)):
        p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(mdir), "--dtype", dt, "--out",
                            str(out), "--max-tokens", "64", "--page-size", "4"], input="\n".join(json.dumps(s) for s in steps),
                           capture_output=True, text=True, timeout=300)
        assert p.returncode == 0, p.stderr[-2000:]
        assert [ln for ln in p.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(7)]
        f32 = {k: v.float() for k, v in sd.items()}
        wa, wb = (_oracle_logits(cfgd, f32, t, torch.float32 if dt == "float32" else torch.bfloat16) for t in (a, b))
        import numpy as np
        got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(3, V))
        assert rel_err(got0, torch.stack([wa[0], wa[19], wb[4]])) < tol
        got2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(1, V))       # b wanted nothing in step 2
        assert rel_err(got2, wa[21:22]) < tol
        got3 = torch.from_numpy(np.fromfile(out / "3.f32", dtype="<f4").reshape(2, V))
        assert rel_err(got3, torch.stack([wa[22], wb[7]])) < tol
        got6 = torch.from_numpy(np.fromfile(out / "6.f32", dtype="<f4").reshape(1, V))
        assert rel_err(got6, wa[25:26]) < tol
