"""The Fidizen design on the HIP path against the plain oracle (oracle/seqmix.py): its mechanisms alone through their own
entry points of libumbrella_seq.so (input convolution with state, PolyNorm, expert routing with the grouped product, latent
attention with window, sink and gate), then whole models through the runtime, the cache manager, the batch engine and the
trace replay command.

fp32 runs are the sharp ones (every comparison to ~1e-5: one key too many or too few in a softmax over a few dozen keys is a
thousand times that); bf16 runs use inputs built so that a fault still shows."""
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


def i32(v):
    return torch.tensor(v, dtype=torch.int32, device="cuda:0")


def close(got, want, tol):
    got, want = got.double().cpu(), want.double().cpu()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30)) < tol


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()).max())


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


# ------------------------------------------------------------------ linear variants
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,N,K,B", [(1, 12, 8, 3), (5, 9, 6, 2), (37, 20, 32, 5), (70, 72, 136, 2)])
def test_batched_linear_with_strides_and_gate(lib, dtype, T, N, K, B):
    from umbrella_amd import _lib
    g = torch.Generator().manual_seed(T + N)
    ldx, ldo = B * K + 8, B * N + 3
    x = torch.randn(T, ldx, generator=g).to(dtype)
    w = (torch.randn(B, N, K, generator=g) / K ** 0.5).to(dtype)
    gate = torch.randn(T, B * N + 5, generator=g)
    xs = torch.stack([x[:, b * K:(b + 1) * K] for b in range(B)]).double()
    want = torch.einsum("btk,bnk->tbn", xs, w.double())
    out = torch.zeros(T, ldo, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_seq_linear_batched", out, dev(x), dev(w), T, N, K, ldx, ldo, B, K, N * K, N, 0, None, 0, 0, _lib.seq_dtype_code(dtype))
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert close(out[:, :B * N].reshape(T, B, N), want, tol) and float(out[:, B * N:].abs().max()) == 0.0
    outg = torch.zeros(T, ldo, dtype=dtype, device="cuda:0")
    _lib.seq_call("umb_seq_linear_batched", outg, dev(x), dev(w), T, N, K, ldx, ldo, B, K, N * K, N, 3, dev(gate), gate.shape[1], N,
                  _lib.seq_dtype_code(dtype))
    wantg = want * torch.sigmoid(gate[:, :B * N].double()).reshape(T, B, N)
    assert close(outg[:, :B * N].reshape(T, B, N), wantg, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_grouped_linear_walks_a_tile_list(lib, dtype):
    from umbrella_amd import _lib
    g = torch.Generator().manual_seed(2)
    G, N, K = 4, 72, 40
    x = torch.randn(150, K, generator=g).to(dtype)
    w = (torch.randn(G, 2 * N, K, generator=g) / K ** 0.5).to(dtype)
    tiles = [(2, 0, 64), (2, 64, 6), (0, 70, 1), (3, 71, 64), (0, 0, 0), (1, 135, 15)]
    grp = torch.zeros(150, dtype=torch.long)
    for e, r0, n in tiles:
        grp[r0:r0 + n] = e
    out = torch.zeros(150, 2 * N, dtype=torch.float32, device="cuda:0")
    code = _lib.seq_dtype_code(dtype)
    _lib.seq_call("umb_seq_linear_grouped", out, dev(x), dev(w), i32(tiles), len(tiles), 64, 2 * N * K, 2 * N, K, 0, code)
    want = torch.einsum("tk,tnk->tn", x.double(), w.double()[grp])
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert close(out, want, tol)
    act = torch.zeros(150, N, dtype=dtype, device="cuda:0")
    _lib.seq_call("umb_seq_linear_grouped", act, dev(x), dev(w), i32(tiles), len(tiles), 64, 2 * N * K, 2 * N, K, 2, code)
    assert close(act, torch.nn.functional.silu(want[:, :N]) * want[:, N:], tol)
    small = [(3, 10, 16), (0, 26, 1), (1, 27, 5), (2, 0, 0)]          # tiles of up to 16 rows: one output tile per workgroup
    out.zero_()
    _lib.seq_call("umb_seq_linear_grouped", out, dev(x), dev(w), i32(small), len(small), 16, 2 * N * K, 2 * N, K, 0, code)
    g16 = torch.zeros(150, dtype=torch.long)
    g16[10:26], g16[26], g16[27:32] = 3, 0, 1
    w16 = torch.einsum("tk,tnk->tn", x.double(), w.double()[g16])
    assert close(out[10:32], w16[10:32], tol) and float(out[:10].abs().max()) == 0.0 and float(out[32:].abs().max()) == 0.0
    if dtype != torch.float32:               # tiles of up to 128 rows on the LDS-staged kernel
        big = [(1, 0, 128), (3, 128, 22), (0, 0, 0)]
        grp[:128], grp[128:150] = 1, 3
        want = torch.einsum("tk,tnk->tn", x.double(), w.double()[grp])
        out.zero_(), act.zero_()
        _lib.seq_call("umb_seq_linear_grouped", out, dev(x), dev(w), i32(big), len(big), 128, 2 * N * K, 2 * N, K, 0, code)
        assert close(out, want, tol)
        _lib.seq_call("umb_seq_linear_grouped", act, dev(x), dev(w), i32(big), len(big), 128, 2 * N * K, 2 * N, K, 2, code)
        assert close(act, torch.nn.functional.silu(want[:, :N]) * want[:, N:], tol)


# ------------------------------------------------------------------ input convolution
def _run_conv(lib, x, w, taps, splits, state, slot, dtype=torch.float32):
    """one sequence in portions: convolution then state update per step (one launch when the step is a single token)"""
    from umbrella_amd import _lib
    n, W = x.shape
    out, at = [], 0
    code = _lib.seq_dtype_code(dtype)
    for k in splits:
        xs = dev(x[at:at + k], torch.float32)
        h = torch.zeros(k, W, dtype=dtype, device="cuda:0")
        pos, sl = i32(list(range(at, at + k))), i32([slot] * k)
        if k == 1:
            _lib.seq_call("umb_canon_step", h, xs, w, state, pos, sl, k, W, taps, code)
        else:
            _lib.seq_call("umb_canon_conv", h, xs, w, state, pos, sl, k, W, taps, code)
            _lib.seq_call("umb_canon_update", state, xs, i32([slot]), i32([0]), i32([at]), i32([k]), 1, W, taps)
        out.append(h.clone())
        at += k
    return torch.cat(out)


@pytest.mark.parametrize("taps,W", [(1, 20), (2, 33), (4, 64), (5, 300)])
def test_input_convolution_in_portions_and_reused_slots(lib, taps, W):
    from oracle import seqmix as O
    g = torch.Generator().manual_seed(taps)
    n = 23
    x, w = torch.randn(n, W, generator=g), torch.randn(W, taps, generator=g)
    want = O.conv_input(x.double(), w.double())
    state = torch.full((3, max(taps - 1, 1), W), 1e6, dtype=torch.float32, device="cuda:0")     # what a used slot may hold
    for slot, splits in ((1, [n]), (1, [1] * n), (2, [2, 2, 1, 5, 1, 1, 3, 8]), (1, [3, 1, 1, 2, 16]), (0, [7, 16])):
        got = _run_conv(lib, x, dev(w), taps, splits, state, slot)
        assert close(got, want, 1e-6), (slot, splits)
    # the first tokens see zeros before the sequence's start, not what the slot held
    assert close(got[0], x[0].double() * (1 + w[:, -1].double()), 1e-6)


def test_input_convolution_batch_of_unequal_sequences(lib):
    from oracle import seqmix as O
    from umbrella_amd import _lib
    g = torch.Generator().manual_seed(9)
    W, taps = 48, 4
    xa, xb, w = torch.randn(9, W, generator=g), torch.randn(4, W, generator=g), torch.randn(W, taps, generator=g)
    state = torch.zeros(4, taps - 1, W, dtype=torch.float32, device="cuda:0")
    wd = dev(w)
    # step 1: a brings 6 tokens, b brings 1; step 2: a brings 3 more, b brings 3 more
    got = {"a": [], "b": []}
    for (na0, na), (nb0, nb) in (((0, 6), (0, 1)), ((6, 3), (1, 3))):
        x = dev(torch.cat([xa[na0:na0 + na], xb[nb0:nb0 + nb]]))
        h = torch.zeros(na + nb, W, dtype=torch.float32, device="cuda:0")
        pos, sl = i32(list(range(na0, na0 + na)) + list(range(nb0, nb0 + nb))), i32([3] * na + [0] * nb)
        _lib.seq_call("umb_canon_conv", h, x, wd, state, pos, sl, na + nb, W, taps, 2)
        _lib.seq_call("umb_canon_update", state, x, i32([3, 0]), i32([0, na]), i32([na0, nb0]), i32([na, nb]), 2, W, taps)
        got["a"].append(h[:na].clone()), got["b"].append(h[na:].clone())
    assert close(torch.cat(got["a"]), O.conv_input(xa.double(), w.double()), 1e-6)
    assert close(torch.cat(got["b"]), O.conv_input(xb.double(), w.double()), 1e-6)


@pytest.mark.parametrize("taps,W,groups", [(1, 40, 1), (2, 300, 1), (4, 2048, 1), (3, 1024, 2), (7, 520, 1)])
def test_seam_with_convolution_in_one_launch(lib, taps, W, groups):
    """single-token steps: x += norm(y) * w, h = conv(x), state update -- against the oracle over a whole sequence"""
    from oracle import seqmix as O
    from umbrella_amd import _lib
    assert lib.umb_seq_resid_canon_step_ok(W, groups) == 1 and lib.umb_seq_resid_canon_step_ok(300, 3) == 0
    g = torch.Generator().manual_seed(W)
    n, eps = 9, 1e-5
    x0, y = torch.randn(n, W, generator=g), torch.randn(n, W, generator=g)
    w_post, w = 1 + 0.1 * torch.randn(W, generator=g), torch.randn(W, taps, generator=g)
    x_want = x0.double() + O.group_rms_norm(y.double(), w_post.double(), groups, eps)
    h_want = O.conv_input(x_want, w.double())
    state = torch.full((2, max(taps - 1, 1), W), 1e6, dtype=torch.float32, device="cuda:0")
    wd, wp = dev(w), dev(w_post)
    for t in range(n):
        x, h = dev(x0[t:t + 1]), torch.zeros(1, W, dtype=torch.float32, device="cuda:0")
        _lib.seq_call("umb_seq_resid_canon_step", x, h, dev(y[t:t + 1]), wp, wd, state, i32([t]), i32([1]), 1, W, groups, taps, eps, 2)
        assert close(x, x_want[t:t + 1], 1e-6) and close(h, h_want[t:t + 1], 1e-5), t


# ------------------------------------------------------------------ feed-forward pieces
@pytest.mark.parametrize("T,F", [(1, 7), (5, 256), (3, 1000)])
def test_polynorm(lib, T, F):
    from oracle import seqmix as O
    from umbrella_amd import _lib
    g = torch.Generator().manual_seed(F)
    z, coef = 2.0 * torch.randn(T, F, generator=g), torch.tensor([0.7, -0.4, 0.2, 0.05])
    out = torch.zeros(T, F, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_polynorm", out, dev(z), dev(coef), T, F, 1e-5, 2)
    assert close(out, O.polynorm(z.double(), coef.double(), 1e-5), 1e-5)


def _run_experts(lib, X, w_router, experts, top, shared, dtype, tile_rows=64):
    """the steps of a routed feed-forward through the library's entry points"""
    from umbrella_amd import _lib
    T, W = X.shape
    E, Fe = len(experts), experts[0][0].shape[0]
    code = _lib.seq_dtype_code(dtype)
    h = dev(X, dtype)
    logits = torch.zeros(T, E, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_seq_linear", logits, h, dev(w_router, dtype), None, T, E, W, 0, code)
    pairs, max_tiles = T * top, (T * top + tile_rows - 1) // tile_rows + E
    sel, wt = torch.zeros(pairs, dtype=torch.int32, device="cuda:0"), torch.zeros(pairs, dtype=torch.float32, device="cuda:0")
    pos, tiles = torch.zeros(pairs, dtype=torch.int32, device="cuda:0"), torch.full((max_tiles, 3), -7, dtype=torch.int32, device="cuda:0")
    _lib.seq_call("umb_moe_route", sel, wt, logits, T, E, top)
    _lib.seq_call("umb_moe_plan", pos, tiles, sel, T, E, top, max_tiles, tile_rows)
    assert sorted(pos.tolist()) == list(range(pairs))                    # every pair has a row of its own
    xs = torch.zeros(pairs, W, dtype=dtype, device="cuda:0")
    _lib.seq_call("umb_moe_scatter", xs, h, wt, pos, T, W, top, code)
    e_gu = dev(torch.stack([torch.cat([g_, u_]) for g_, u_, _ in experts]), dtype)
    e_down = dev(torch.stack([d_ for _, _, d_ in experts]), dtype)
    act = torch.zeros(pairs, Fe, dtype=dtype, device="cuda:0")
    ye = torch.zeros(pairs, W, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_seq_linear_grouped", act, xs, e_gu, tiles, max_tiles, tile_rows, 2 * Fe * W, 2 * Fe, W, 2, code)
    _lib.seq_call("umb_seq_linear_grouped", ye, act, e_down, tiles, max_tiles, tile_rows, W * Fe, W, Fe, 0, code)
    y = torch.full((T, W), 5.0, dtype=torch.float32, device="cuda:0")
    if shared is not None:
        Fs = shared[0].shape[0]
        a2 = torch.zeros(T, Fs, dtype=dtype, device="cuda:0")
        _lib.seq_call("umb_seq_linear", a2, h, dev(torch.cat([shared[0], shared[1]]), dtype), None, T, 2 * Fs, W, 2, code)
        _lib.seq_call("umb_seq_linear", y, a2, dev(shared[2], dtype), None, T, W, Fs, 0, code)
    _lib.seq_call("umb_moe_combine", y, ye, pos, T, W, top, 1 if shared is not None else 0)
    return y, sel.reshape(T, top), wt.reshape(T, top)


@pytest.mark.parametrize("T,W,E,top,Fe,Fs", [(1, 24, 4, 1, 8, 0), (50, 40, 5, 2, 12, 10), (200, 32, 70, 4, 16, 8), (33, 36, 3, 3, 5, 7)])
def test_routed_experts_against_oracle(lib, T, W, E, top, Fe, Fs):
    from oracle import seqmix as O
    g = torch.Generator().manual_seed(E * 10 + top)
    X = torch.randn(T, W, generator=g)
    w_router = 3.0 * torch.randn(E, W, generator=g) / W ** 0.5
    ex = [(torch.randn(Fe, W, generator=g) / W ** 0.5, torch.randn(Fe, W, generator=g) / W ** 0.5,
           torch.randn(W, Fe, generator=g) / Fe ** 0.5) for _ in range(E)]
    sh = (torch.randn(Fs, W, generator=g) / W ** 0.5, torch.randn(Fs, W, generator=g) / W ** 0.5,
          torch.randn(W, Fs, generator=g) / Fs ** 0.5) if Fs else None
    y, sel, wt = _run_experts(lib, X, w_router, ex, top, sh, torch.float32)
    d = lambda t: tuple(v.double() for v in t)
    want = O.routed_experts(X.double(), w_router.double(), [d(e) for e in ex], top, d(sh) if sh else None)
    assert close(y, want, 2e-5)
    s = torch.sigmoid(X.double() @ w_router.double().T)
    assert close(wt, s.gather(1, sel.cpu().long()), 1e-5)                    # the weights are the scores themselves


def test_routed_experts_many_rows_per_expert_in_16_bits(lib):
    """bf16, 600 tokens over 3 experts: tiles of 128 rows on the LDS-staged grouped kernel against tiles of 64"""
    g = torch.Generator().manual_seed(4)
    T, W, E, top, Fe = 600, 64, 3, 2, 40
    X = torch.randn(T, W, generator=g)
    w_router = 3.0 * torch.randn(E, W, generator=g) / W ** 0.5
    ex = [(torch.randn(Fe, W, generator=g) / W ** 0.5, torch.randn(Fe, W, generator=g) / W ** 0.5,
           torch.randn(W, Fe, generator=g) / Fe ** 0.5) for _ in range(E)]
    a, sel_a, _ = _run_experts(lib, X, w_router, ex, top, None, torch.bfloat16, tile_rows=64)
    b, sel_b, _ = _run_experts(lib, X, w_router, ex, top, None, torch.bfloat16, tile_rows=128)
    assert torch.equal(sel_a, sel_b) and close(b, a, 1e-2)
    from oracle import seqmix as O
    r = lambda t: t.to(torch.bfloat16).double()
    want = O.routed_experts(r(X), r(w_router), [tuple(r(v) for v in e) for e in ex], top)
    bad = (b.double().cpu() - want).abs().max(-1).values > 0.05 * want.abs().max()
    assert int(bad.sum()) <= 6               # a handful of tokens may sit on a routing tie that 16-bit inputs flip


def test_routing_breaks_ties_by_index_and_one_token_does_not_move_another(lib):
    from umbrella_amd import _lib
    T, E, top = 6, 9, 3
    logits = torch.zeros(T, E)
    logits[1, 4] = logits[1, 7] = 2.0                     # two equal leaders, the rest equal
    logits[2] = torch.arange(E).float()
    sel, wt = torch.zeros(T * top, dtype=torch.int32, device="cuda:0"), torch.zeros(T * top, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_moe_route", sel, wt, dev(logits), T, E, top)
    sel = sel.reshape(T, top).tolist()
    assert sel[0] == [0, 1, 2] and sel[1] == [4, 7, 0] and sel[2] == [8, 7, 6]


# ------------------------------------------------------------------ latent attention alone
def _lat_weights(width, H, D, R, E, q_rank, kv_rank, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g) / s[-1] ** 0.5
    return dict(dq=r(q_rank, width), dq_n=1 + 0.1 * torch.randn(q_rank, generator=g), uq=r(H * (D + R), q_rank),
                dkv=r(kv_rank + R, width), dkv_n=1 + 0.1 * torch.randn(kv_rank, generator=g), uk=r(H * D, kv_rank),
                uv=r(H * E, kv_rank), sink=torch.randn(H, generator=g), g=r(H * E, width), o=r(width, H * E))


def _run_latent(lib, X, w, *, H, D, R, E, q_rank, kv_rank, window, rot_dims, base, scale, eps, dtype, page, splits, cache=None,
                seq="s"):
    """the mixer's steps through the library's entry points, the sequence fed in portions"""
    from umbrella_amd import _lib
    from umbrella_amd.attn.cache import PagedSeqCache
    n, width = X.shape
    code, Dk = _lib.seq_dtype_code(dtype), kv_rank + R
    cache = cache or PagedSeqCache([], [], max_tokens=n + 2 * page, max_seqs=2, device="cuda:0", dtype=dtype, page=page, latent_layers=[Dk])
    cache.open(seq)
    kv = cache.latent_struct(0)
    wd = {k: dev(v, dtype) for k, v in w.items()}
    proj_w = torch.cat([wd["dq"], wd["dkv"], wd["g"]])
    uk_t = wd["uk"].view(H, D, kv_rank).transpose(1, 2).contiguous()
    freq = dev(base ** (-2 * torch.arange(rot_dims // 2, dtype=torch.float32) / rot_dims)) if rot_dims else None
    ld, f32 = proj_w.shape[0], torch.float32
    out, at = [], 0
    for k in splits:
        p0 = cache.extend(seq, k)
        sl = cache.slot(seq)
        pos, slot = i32(list(range(p0, p0 + k))), i32([sl] * k)
        z = lambda *s, dt=f32: torch.zeros(*s, dtype=dt, device="cuda:0")
        h, proj, cq, q, qn, qa = dev(X[at:at + k], dtype), z(k, ld), z(k, q_rank, dt=dtype), z(k, H * (D + R)), z(k, H * D, dt=dtype), z(k, H * Dk)
        ol, mix, y = z(k, H * kv_rank, dt=dtype), z(k, H * E, dt=dtype), z(k, width)
        _lib.seq_call("umb_seq_linear", proj, h, proj_w, None, k, ld, width, 0, code)
        _lib.seq_call("umb_lat_prep", cq, kv, proj, ld, wd["dq_n"], wd["dkv_n"], pos, slot, freq, k, q_rank, kv_rank, R, rot_dims, eps, code)
        _lib.seq_call("umb_seq_linear", q, cq, wd["uq"], None, k, H * (D + R), q_rank, 0, code)
        _lib.seq_call("umb_lat_qsplit", qn, qa, q, pos, freq, k, H, D, R, kv_rank, rot_dims, code)
        _lib.seq_call("umb_seq_linear_batched", qa, qn, uk_t, k, kv_rank, D, H * D, H * Dk, H, D, kv_rank * D, Dk, 0, None, 0, 0, code)
        if k >= 16 and _lib.load_seq().umb_lat_attend_tiled_ok(H, kv_rank, R, code):
            _lib.seq_call("umb_lat_attend_tiled", ol, qa, kv, wd["sink"], i32([sl]), i32([0]), i32([p0]), i32([k]), 1, k, H, kv_rank, R,
                          window or 2 ** 30, scale, code)
        else:
            _lib.seq_call("umb_lat_attend", ol, qa, kv, wd["sink"], pos, slot, k, H, kv_rank, R, window or 2 ** 30, scale, code)
        _lib.seq_call("umb_seq_linear_batched", mix, ol, wd["uv"], k, E, kv_rank, H * kv_rank, H * E, H, kv_rank, E * kv_rank, E, 3,
                      proj[:, q_rank + Dk:], ld, E, code)
        _lib.seq_call("umb_seq_linear", y, mix, wd["o"], None, k, width, H * E, 0, code)
        out.append(y.clone())
        at += k
    return torch.cat(out), cache


def _lat_oracle(X, w, dtype, **kw):
    from oracle import seqmix as O
    r = None if dtype == torch.float32 else (lambda t: t.to(dtype).double())
    d = {k: v.to(dtype).double() for k, v in w.items()}
    return O.latent_attention(X.to(dtype).double(), d["dq"], d["dq_n"], d["uq"], d["dkv"], d["dkv_n"], d["uk"], d["uv"], d["sink"],
                              d["g"], d["o"], cache_round=r, **kw)


LAT_CASES = [  # H, D, R, E, q_rank, kv_rank, window, rot_dims, page
    (3, 8, 4, 6, 10, 12, 5, 4, 4), (5, 6, 6, 10, 7, 9, 1, 4, 3), (1, 3, 2, 5, 3, 70, 4, 2, 5), (9, 16, 8, 24, 48, 136, 70, 8, 16),
    (2, 32, 16, 8, 24, 264, 0, 16, 64), (4, 16, 0, 16, 8, 32, 7, 0, 4), (16, 8, 8, 8, 16, 64, 33, 8, 8), (3, 8, 8, 8, 16, 600, 20, 8, 8)]


@pytest.mark.parametrize("H,D,R,E,q_rank,kv_rank,window,rot_dims,page", LAT_CASES)
def test_latent_attention_alone_every_position(lib, H, D, R, E, q_rank, kv_rank, window, rot_dims, page):
    """fp32, every position of a sequence longer than the window and several pages, whole and in portions down to one token"""
    width, n = 40, 90
    w = _lat_weights(width, H, D, R, E, q_rank, kv_rank, seed=H * 7 + D)
    X = torch.randn(n, width, generator=torch.Generator().manual_seed(1))
    kw = dict(H=H, D=D, R=R, E=E, kv_rank=kv_rank, window=window, rot_dims=rot_dims, base=50.0, scale=0.3, eps=1e-5)
    want = _lat_oracle(X, w, torch.float32, **kw)
    for splits in ([n], [1] * n, [2, 2, 17, 1, 40, 3, 25]):
        got, _ = _run_latent(lib, X, w, q_rank=q_rank, dtype=torch.float32, page=page, splits=splits, **kw)
        assert close(got, want, F32_TOL), splits


MFMA_CASES = [  # H, D, R, E, q_rank, kv_rank, window, rot_dims, page: key rows that are and are not multiples of 32 features
    (4, 16, 8, 16, 24, 32, 6, 8, 4), (9, 16, 16, 24, 48, 144, 70, 16, 16), (2, 32, 24, 8, 24, 272, 0, 16, 64),
    (16, 8, 8, 8, 16, 64, 33, 8, 5), (3, 8, 24, 12, 16, 80, 1, 4, 3), (8, 16, 0, 16, 8, 16, 20, 0, 7)]


@pytest.mark.parametrize("single", ["vector", "matrix"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("H,D,R,E,q_rank,kv_rank,window,rot_dims,page", MFMA_CASES)
def test_latent_attention_on_the_matrix_pipe(lib, monkeypatch, single, dtype, H, D, R, E, q_rank, kv_rank, window, rot_dims, page):
    """16-bit storage: prompt portions of 16 tokens and more take the matrix-pipe kernel (tiles that start inside a window,
    end before a full tile, span pages); shorter ones the vector-pipe kernel or, from a few dozen tokens a step (here: forced),
    the matrix-pipe kernel whose query tile is sixteen heads of one token; all against the oracle and against each other"""
    from umbrella_amd import _lib
    monkeypatch.setenv("UMB_LAT_DEC_MIN", "0" if single == "matrix" else "1000000")
    assert lib.umb_lat_attend_tiled_ok(H, kv_rank, R, _lib.seq_dtype_code(dtype)) == 1
    width, n = 40, 100
    w = _lat_weights(width, H, D, R, E, q_rank, kv_rank, seed=H + kv_rank)
    X = torch.randn(n, width, generator=torch.Generator().manual_seed(2))
    kw = dict(H=H, D=D, R=R, E=E, kv_rank=kv_rank, window=window, rot_dims=rot_dims, base=50.0, scale=0.3, eps=1e-5)
    want = _lat_oracle(X, w, dtype, **kw)
    tol = BF16_TOL if dtype == torch.bfloat16 else 1e-2
    outs = []
    for splits in ([n], [17, 16, 3, 33, 31], [1] * 12 + [88]):
        got, _ = _run_latent(lib, X, w, q_rank=q_rank, dtype=dtype, page=page, splits=splits, **kw)
        assert close(got, want, tol), splits
        outs.append(got)
    assert close(outs[1], outs[0], tol / 2) and close(outs[2], outs[0], tol / 2)


def _loud(n, width, rows, seed):
    """inputs whose rows `rows` are thirty times the others: their rotated key part (it is not normed) dominates every
    score it enters, so a window one token off moves the output of about every other head completely"""
    X = torch.randn(n, width, generator=torch.Generator().manual_seed(seed))
    for r in rows:
        X[r] *= 30.0
    return X


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_latent_window_edges_and_far_keys_with_loud_rows(lib, monkeypatch, dtype):
    """loud keys just inside and just outside the window of the last positions, at a page border and far back, in a prompt
    and in token-by-token decoding; the softmax spans hundreds of keys"""
    if dtype == torch.float16:                       # this run decodes single tokens on the matrix pipe
        monkeypatch.setenv("UMB_LAT_DEC_MIN", "0")
    H, D, R, E, q_rank, kv_rank, window, page = 4, 16, 8, 16, 24, 48, 150, 32
    width, n = 48, 260
    w = _lat_weights(width, H, D, R, E, q_rank, kv_rank, seed=5)
    kw = dict(H=H, D=D, R=R, E=E, kv_rank=kv_rank, window=window, rot_dims=8, base=1000.0, scale=0.2, eps=1e-5)
    tol = F32_TOL if dtype == torch.float32 else (BF16_TOL if dtype == torch.bfloat16 else 1e-2)
    for rows in ([n - window], [n - window - 1], [n - 1 - window, 3], [0, 31, 32, n - window + 1], [n - 20 - window, n - 21 - window]):
        X = _loud(n, width, rows, seed=len(rows))
        want = _lat_oracle(X, w, dtype, **kw)
        for splits in ([n], [n - 40] + [1] * 40):
            got, _ = _run_latent(lib, X, w, q_rank=q_rank, dtype=dtype, page=page, splits=splits, **kw)
            assert close(got[-45:], want[-45:], tol), (rows, splits[:2])
    # the loud key matters: moving it across the edge changes what the last position reads
    a = _lat_oracle(_loud(n, width, [n - window], 1), w, torch.float32, **kw)[-1]
    b = _lat_oracle(_loud(n, width, [n - window - 1], 1), w, torch.float32, **kw)[-1]
    assert float((a - b).abs().max() / a.abs().max()) > 0.05


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_sink_takes_weight_without_a_value(lib, dtype):
    H, D, R, E, q_rank, kv_rank = 2, 8, 4, 8, 8, 16
    width, n = 32, 12
    kw = dict(H=H, D=D, R=R, E=E, kv_rank=kv_rank, window=6, rot_dims=4, base=100.0, scale=0.3, eps=1e-5)
    w = _lat_weights(width, H, D, R, E, q_rank, kv_rank, seed=8)
    X = torch.randn(n, width, generator=torch.Generator().manual_seed(3))
    outs = {}
    for s in (-30.0, 0.0, 12.0):
        w["sink"] = torch.tensor([s, s - 1.0])
        got, _ = _run_latent(lib, X, w, q_rank=q_rank, dtype=dtype, page=4, splits=[5, 1, 1, 5], **kw)
        assert close(got, _lat_oracle(X, w, dtype, **kw), F32_TOL if dtype == torch.float32 else BF16_TOL), s
        outs[s] = got
    assert float(outs[12.0].abs().max()) < 0.01 * float(outs[-30.0].abs().max())       # a large sink swallows the weights


def test_latent_pages_are_reused_without_leaking(lib):
    """a long sequence fills pages with loud rows, ends, and a second one gets the same pages and slot"""
    from umbrella_amd.attn.cache import PagedSeqCache
    H, D, R, E, q_rank, kv_rank, page = 3, 8, 4, 6, 10, 12, 4
    width = 40
    kw = dict(H=H, D=D, R=R, E=E, kv_rank=kv_rank, window=9, rot_dims=4, base=50.0, scale=0.3, eps=1e-5)
    w = _lat_weights(width, H, D, R, E, q_rank, kv_rank, seed=2)
    cache = PagedSeqCache([], [], max_tokens=40, max_seqs=1, device="cuda:0", dtype=torch.float32, page=page, latent_layers=[kv_rank + R])
    X1 = 50.0 * torch.randn(37, width, generator=torch.Generator().manual_seed(1))
    _run_latent(lib, X1, w, q_rank=q_rank, dtype=torch.float32, page=page, splits=[37], cache=cache, seq="one", **kw)
    first = list(cache.seqs["one"]["pages"])
    cache.close("one")
    X2 = torch.randn(30, width, generator=torch.Generator().manual_seed(2))
    got, _ = _run_latent(lib, X2, w, q_rank=q_rank, dtype=torch.float32, page=page, splits=[3, 1, 1, 25], cache=cache, seq="two", **kw)
    assert cache.seqs["two"]["pages"] == first[:len(cache.seqs["two"]["pages"])]
    assert close(got, _lat_oracle(X2, w, torch.float32, **kw), F32_TOL)


# ------------------------------------------------------------------ whole models
def _oracle_logits(cfgd, sd, toks, dtype, margins=None):
    from oracle import seqmix as O
    r = None if dtype == torch.float32 else (lambda t: t.to(dtype).double())
    return O.fidizen_forward(cfgd, sd, toks, cache_round=r, route_margins=margins)


def _calm_tokens(cfgd, sd, n, dtype, seed0=5):
    """a token sequence whose expert choices stand clear of every runner-up (16-bit runs drift by a percent: a choice that
    hangs on less would make the test one of rounding, not of the mechanism) -> (tokens, the oracle's logits)"""
    for seed in range(seed0, seed0 + 200):
        toks, margins = tokens(n, cfgd["vocab"], seed), []
        want = _oracle_logits(cfgd, sd, toks, dtype, margins)
        if dtype == torch.float32 or not margins or min(margins) > 0.03:
            return toks, want
    raise AssertionError("no calm token sequence found")


def _few_experts(cfgd):
    """the same shape with at most six experts of which at most two are used (for 16-bit runs)"""
    out = json.loads(json.dumps(cfgd))
    for ly in out["layers"]:
        if ly["mlp"] and ly["mlp"]["kind"] == "moe" and ly["mlp"]["router"]["experts"] > 8:
            ly["mlp"]["router"] = {"experts": 6, "top": 2}
    return out


@pytest.mark.parametrize("name", ["mixed", "odd", "wide", "one_tap"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_prefill_decode_portions_against_oracle(lib, name, dtype):
    from fidizen_helpers import CONFIGS, build
    cfgd = CONFIGS[name] if dtype == torch.float32 else _few_experts(CONFIGS[name])
    m, sd = build(cfgd, dtype, seed=11, page=4)
    n = 41
    toks, want = _calm_tokens(cfgd, sd, n, dtype)
    tol = F32_TOL if dtype == torch.float32 else BF16_TOL
    m.open("w")
    whole, layers = m.forward_batch([("w", toks)], want=[list(range(n))], trace=True)
    whole = whole.clone()
    if dtype == torch.float32:                      # the residual stream after every layer, shared layers counted each time
        from oracle import seqmix as O
        lo = []
        O.fidizen_forward(cfgd, sd, toks, layers_out=lo)
        assert layers.shape[0] == len(cfgd["layers"]) and close(layers, torch.stack(lo), F32_TOL)
    assert rel_err(whole, want) < tol
    same = F32_TOL if dtype == torch.float32 else 2e-2          # the model against itself under another schedule
    for sid, splits in (("d", [1] * n), ("p", [2, 2, 7, 1, 16, 3, 10]), ("q", [30] + [1] * 11), ("r", [17, 2, 2, 20])):
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
    from fidizen_helpers import CONFIGS, build
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


def test_model_sixty_sequences_decoded_together(lib):
    """bf16: sixty requests of different lengths, prefilled in one ragged step and decoded together for a few steps (steps of
    sixty single tokens take the matrix-pipe kernel for single tokens), against each request alone"""
    from fidizen_helpers import CONFIGS, build
    cfgd = _few_experts(CONFIGS["wide"])
    m, _ = build(cfgd, torch.bfloat16, seed=5, page=8, batch=61, max_tokens=4000)
    V = cfgd["vocab"]
    seqs = {k: tokens(4 + (7 * k) % 40, V, 100 + k) for k in range(60)}
    for k in seqs:
        m.open(k)
    got = {k: [] for k in seqs}
    out = m.forward_batch([(k, t[:-3]) for k, t in seqs.items()]).clone()          # the last row of each
    for i, k in enumerate(seqs):
        got[k].append(out[i:i + 1])
    for step in range(3):
        out = m.forward_batch([(k, [t[len(t) - 3 + step]]) for k, t in seqs.items()]).clone()
        for i, k in enumerate(seqs):
            got[k].append(out[i:i + 1])
    worst = 0.0
    for k, t in list(seqs.items())[::7]:
        m.open("solo")
        n = len(t)
        alone = m.forward_batch([("solo", t)], want=[[n - 4, n - 3, n - 2, n - 1]]).clone()
        m.close("solo")
        worst = max(worst, rel_err(torch.cat(got[k]), alone))
    assert worst < 3e-2, worst


def test_model_long_decoding_past_the_window_and_first_tokens(lib):
    """fp32: 150 tokens decoded one by one after a two-token prompt (windows of 5, 9 and none; pages of 4 tokens used up and
    down the table) against the oracle's whole-sequence pass; the first positions see nothing before them"""
    from fidizen_helpers import CONFIGS, build
    cfgd = CONFIGS["mixed"]
    m, sd = build(cfgd, torch.float32, seed=7, page=4, batch=2, max_tokens=400)
    toks = tokens(152, cfgd["vocab"], seed=9)
    want = _oracle_logits(cfgd, sd, toks, torch.float32)
    m.open("x")
    rows = [m.forward_batch([("x", toks[:2])], want=[[0, 1]]).clone()]
    for t in toks[2:]:
        rows.append(m.forward_batch([("x", [t])], want=[[0]]).clone())
    got = torch.cat(rows)
    assert rel_err(got, want) < F32_TOL
    assert rel_err(got[:3], want[:3]) < F32_TOL


def test_cache_runs_out_loudly_and_recovers(lib):
    from fidizen_helpers import CONFIGS, build
    cfgd = CONFIGS["one_tap"]
    m, _ = build(cfgd, torch.bfloat16, page=4, batch=2, max_tokens=16)
    m.open("a")
    with pytest.raises(RuntimeError):
        m.forward_batch([("a", tokens(40, cfgd["vocab"], 1))])
    m.close("a")
    m.open("b")
    assert m.forward_batch([("b", tokens(10, cfgd["vocab"], 2))]).shape == (1, cfgd["vocab"])


# ------------------------------------------------------------------ engine and command line
def _engine(cfgd, dtype, sd=None, **kw):
    from fidizen_helpers import build
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
        row = O.fidizen_forward(cfgd, sd, toks)[-1]
        top = torch.topk(row, 2).values
        margins.append(float(top[0] - top[1]))
        toks.append(int(row.argmax()))
    return toks[len(prompt):], margins


def test_engine_greedy_generation_matches_oracle(lib):
    """five queued requests through the scheduler (three slots: two batches), greedy, fp32: the oracle's tokens"""
    from fidizen_helpers import CONFIGS
    cfgd = CONFIGS["mixed"]
    e, sd = _engine(cfgd, torch.float32)
    prompts = [tokens(n, cfgd["vocab"], seed=n) for n in (7, 1, 12, 3, 9)]
    outs = e.generate_batch(prompts, max_new_tokens=10)
    for p, got in zip(prompts, outs):
        want, margins = _oracle_greedy(cfgd, sd, p, 10)
        k = next((i for i, (a, b) in enumerate(zip(got, want)) if a != b), None)
        assert k is None or margins[k] < 1e-4, (got, want, margins)
    assert not e.target_model.kv_cache.seqs and len(e.target_model.kv_cache.free_slots) == 3
    api = e.generate(input_ids=prompts[2], max_new_tokens=10)
    assert api["generated_tokens"] == outs[2]


def test_engine_sampling_is_seeded_and_in_range(lib):
    from fidizen_helpers import CONFIGS
    cfgd = CONFIGS["odd"]
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
    import numpy as np
    from safetensors.torch import save_file
    from fidizen_helpers import CONFIGS, checkpoint
    cfgd = CONFIGS["mixed"]
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
        got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(3, V))
        assert rel_err(got0, torch.stack([wa[0], wa[19], wb[4]])) < tol
        got2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(1, V))       # b wanted nothing in step 2
        assert rel_err(got2, wa[21:22]) < tol
        got3 = torch.from_numpy(np.fromfile(out / "3.f32", dtype="<f4").reshape(2, V))
        assert rel_err(got3, torch.stack([wa[22], wb[7]])) < tol
        got6 = torch.from_numpy(np.fromfile(out / "6.f32", dtype="<f4").reshape(1, V))
        assert rel_err(got6, wa[25:26]) < tol
