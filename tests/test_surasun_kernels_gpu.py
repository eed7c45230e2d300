"""Every kernel of the recurrent mixers, of the residual in several streams and of the attention
with capped scores against its plain PyTorch twin (tests/torch_ops.py), at sizes of their own:
packed steps of several sequences of unequal length, states that are continued, rows that lie
apart, sizes that are no multiple of a wavefront."""

import math

import pytest
import torch

import torch_ops as twin
from qwen3_from_scratch_amd import ops

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _rand(g, *shape, scale=1.0, dtype=torch.float32):
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def _step(lengths, slots):
    """cu_seqlens_q, seq_index and slots of a packed step whose sequences bring `lengths` tokens."""
    cu = [0]
    for n in lengths:
        cu.append(cu[-1] + n)
    seq = [b for b, n in enumerate(lengths) for _ in range(n)]
    as_int = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    return as_int(cu), as_int(seq), as_int(slots)


def _close(got, want, tol):
    got, want = got.float(), want.float()
    bound = tol * max(1.0, float(want.abs().max()))
    assert float((got - want).abs().max()) <= bound, (float((got - want).abs().max()), bound)


def _tol(dtype):
    return 2e-5 if dtype == torch.float32 else 1.2e-2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("S,W", [(1, 40), (3, 200), (8, 1030)])
def test_hyper_norm(dtype, S, W):
    g = _gen(S * W)
    T = 7
    x = _rand(g, T, S, W)
    weight, read, write, mix = _rand(g, W), _rand(g, S), _rand(g, S), _rand(g, S, S)
    delta = _rand(g, T, W, dtype=dtype)
    rows = torch.tensor([5, 0, 5, 2], dtype=torch.int32, device=DEV)
    for kwargs in (dict(), dict(read=read), dict(read=read, delta=delta, mix=mix, write=write),
                   dict(delta=delta, mix=mix, write=write, rows=rows), dict(read=read, rows=rows)):
        a, b = x.clone(), x.clone()
        got = ops.hyper_norm(a, weight, 1e-5, dtype, **kwargs)
        want = twin.hyper_norm(b, weight, 1e-5, dtype, **kwargs)
        _close(got, want, _tol(dtype))
        _close(a, b, 1e-5)
    a, b = x.clone(), x.clone()
    assert ops.hyper_norm(a, None, 0.0, dtype, delta=delta, mix=mix, write=write) is None
    twin.hyper_norm(b, None, 0.0, dtype, delta=delta, mix=mix, write=write)
    _close(a, b, 1e-5)
    _close(ops.embed_streams(torch.tensor([3, 1], dtype=torch.int32, device=DEV), delta, S),
           twin.embed_streams(torch.tensor([3, 1], dtype=torch.int32, device=DEV), delta, S), 0.0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,taps,lengths", [(70, 4, [1, 9, 2, 1]), (300, 3, [5, 1, 1, 40]), (64, 2, [3]), (33, 1, [2, 2]),
                                            (80, 4, [1, 1, 1]), (40, 2, [1]), (96, 3, [300, 1, 20]), (64, 4, [2100, 3]),
                                            (4352, 4, [1, 2, 300, 1]), (72, 8, [3, 5, 250]), (100, 2, [260])])
def test_causal_conv_continues_its_state(dtype, C, taps, lengths):
    g = _gen(C + taps)
    wide = _rand(g, sum(lengths), C + (24 if C % 8 == 0 else 25), dtype=dtype)
    x = wide[:, 16:16 + C]
    weight, bias, add = _rand(g, C, taps), _rand(g, C), _rand(g, C)
    cu, seq, slots = _step(lengths, [4, 0, 2, 5][:len(lengths)])
    full = _rand(g, 7, (taps - 1) * C + 10)
    for activation, in_bias, out_dtype in ((None, add, torch.float32), ("silu", None, dtype)):
        a, b = full.clone(), full.clone()
        got = ops.causal_conv(x, weight, bias, a[:, 3:3 + (taps - 1) * C], slots, cu, seq, activation, out_dtype, in_bias,
                              max_q_len=max(lengths))
        want = twin.causal_conv(x, weight, bias, b[:, 3:3 + (taps - 1) * C], slots, cu, seq, activation, out_dtype, in_bias)
        _close(got, want, _tol(out_dtype))
        _close(a, b, 1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,P,N,G,lengths", [(4, 32, 32, 1, [6, 1, 3]), (6, 80, 48, 3, [1, 1]), (2, 16, 130, 2, [9]),
                                             (4, 64, 128, 2, [130, 1, 64, 65]), (3, 72, 24, 1, [200, 7])])
def test_mamba2_scan(dtype, H, P, N, G, lengths):
    g = _gen(H * P + N)
    T = sum(lengths)
    xbc = _rand(g, T, H * P + 2 * G * N, dtype=dtype)
    wide = _rand(g, T, H + 5, dtype=dtype)
    dt = wide[:, 5:]
    dt_bias, a_log, skip = _rand(g, H), _rand(g, H, scale=0.5), _rand(g, H)
    cu, _, slots = _step(lengths, [1, 3, 0, 4][:len(lengths)])
    full = _rand(g, 5, H * N * P + 8, scale=0.3)
    a, b = full.clone(), full.clone()
    got = ops.mamba2_scan(xbc, dt, dt_bias, a_log, skip, a[:, 8:], slots, cu, H, P, N, G, max_q_len=max(lengths))
    want = twin.mamba2_scan(xbc, dt, dt_bias, a_log, skip, b[:, 8:], slots, cu, H, P, N, G)
    _close(got, want, 3e-5)
    _close(a, b, 3e-5)
    if max(lengths) >= ops.CHUNKED_FROM:          # row by row and in chunks: the same results and states
        c = full.clone()
        _close(ops.mamba2_scan(xbc, dt, dt_bias, a_log, skip, c[:, 8:], slots, cu, H, P, N, G, max_q_len=1), got, 3e-5)
        _close(c, a, 3e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,groups", [(128, 1), (120, 3), (640, 5)])
def test_gated_rmsnorm(dtype, n, groups):
    g = _gen(n)
    y, weight = _rand(g, 5, n), _rand(g, n)
    gate = _rand(g, 5, n + 9, dtype=dtype)[:, 4:4 + n]
    _close(ops.gated_rmsnorm(y, gate, weight, groups, 1e-6, dtype), twin.gated_rmsnorm(y, gate, weight, groups, 1e-6, dtype),
           _tol(dtype))


@pytest.mark.parametrize("width,blocks,lengths", [(160, 2, [5, 1, 12]), (96, 3, [1, 1, 1]), (520, 1, [19]),
                                                  (320, 2, [200, 1, 65]), (96, 1, [64, 129]), (2048, 8, [1] * 9),
                                                  (70, 1, [3, 300])])
def test_recurrent_unit_gates_and_recurrence(width, blocks, lengths):
    g = _gen(width)
    T, bw = sum(lengths), width // blocks
    u = _rand(g, T, width)
    weights, biases = _rand(g, 2, blocks, bw, bw, scale=bw ** -0.5), _rand(g, 2, blocks, bw)
    gates = ops.block_gates(u, weights, biases)
    _close(gates, twin.block_gates(u, weights, biases), 2e-5)
    rate = _rand(g, width).abs() + 0.01
    y = _rand(g, T, 2 * width)[:, :width]
    y_bias = _rand(g, width)
    cu, _, slots = _step(lengths, [2, 0, 1, 3, 4, 5, 6, 7, 8][:len(lengths)])
    full = _rand(g, 9, width + 3)
    for dtype in DTYPES:
        a, b = full.clone(), full.clone()
        got = ops.rglru_scan(u, gates, rate, y, y_bias, a[:, 3:], slots, cu, dtype, max_q_len=max(lengths))
        want = twin.rglru_scan(u, gates, rate, y, y_bias, b[:, 3:], slots, cu, dtype)
        _close(got, want, _tol(dtype))
        _close(a, b, 2e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,dim,vdim,rot,lengths", [(4, 64, 64, 64, [7, 1, 2]), (3, 24, 40, 16, [1, 1]), (2, 136, 200, 0, [5]),
                                                    (2, 128, 256, 128, [130, 1, 64]), (3, 40, 72, 20, [100, 65, 3]),
                                                    (1, 200, 96, 64, [70])])
def test_retention_scan(dtype, H, dim, vdim, rot, lengths):
    g = _gen(H * dim + vdim)
    T = sum(lengths)
    rows = _rand(g, T, 2 * H * dim + 2 * H * vdim, dtype=dtype)
    inv_freq = torch.tensor([10000.0 ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32, device=DEV) if rot else None
    first = [100000, 3, 0]
    positions = torch.tensor([first[b] + i for b, n in enumerate(lengths) for i in range(n)], dtype=torch.int32, device=DEV)
    decay = torch.tensor([0.9, 0.99, 0.5, 0.999][:H], dtype=torch.float32, device=DEV)
    cu, _, slots = _step(lengths, [0, 2, 1][:len(lengths)])
    full = _rand(g, 3, H * dim * vdim + 2, scale=0.2)
    a, b = full.clone(), full.clone()
    got = ops.retention_scan(rows, H, dim, vdim, inv_freq, positions, decay, dim ** -0.5, 1e-6, a[:, 2:], slots, cu, dtype,
                             max_q_len=max(lengths))
    want = twin.retention_scan(rows, H, dim, vdim, inv_freq, positions, decay, dim ** -0.5, 1e-6, b[:, 2:], slots, cu, dtype)
    _close(got, want, 2e-3 if dtype == torch.float32 else 2e-2)       # the angle at position 100,000 is a float32 product
    _close(a, b, 1e-4)


def _paged(g, lengths_before, lengths, page, G, dim, vdim, dtype):
    """A cache in which every sequence already holds some tokens, on pages in shuffled order."""
    B = len(lengths)
    totals = [a + b for a, b in zip(lengths_before, lengths)]
    width = max(-(-n // page) for n in totals)
    pages = B * width + 3
    order = torch.randperm(pages, generator=g).tolist()
    table = torch.full((B, width), -1, dtype=torch.int32)
    for b in range(B):
        for i in range(-(-totals[b] // page)):
            table[b, i] = order.pop()
    keys = _rand(g, pages, G, page, dim, dtype=dtype)
    values = _rand(g, pages, G, page, vdim, dtype=dtype)
    positions = torch.tensor([lengths_before[b] + i for b in range(B) for i in range(lengths[b])], dtype=torch.int32, device=DEV)
    return keys, values, table.to(DEV), positions, torch.tensor(totals, dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("transposed", [False, True])
@pytest.mark.parametrize("H,G,dim,vdim,rot,page", [(8, 4, 96, 32, 48, 16), (3, 1, 40, 72, 40, 8), (4, 4, 16, 16, 0, 16),
                                                   (8, 2, 128, 128, 64, 16), (4, 4, 64, 64, 64, 32), (6, 2, 64, 64, 0, 16)])
def test_capped_attention_prepares_and_attends(dtype, H, G, dim, vdim, rot, page, transposed):
    """Both layouts of the values; with transposed values, bfloat16 and equal sizes of 64 or 128 the
    matrix-core kernels run (the last three cases), else the general one."""
    g = _gen(H * dim + vdim)
    before, lengths = [37, 0, 130], [5, 21, 1] if dim != 128 else [5, 150, 1]
    T = sum(lengths)
    keys, values, table, positions, kv_lens = _paged(g, before, lengths, page, G, dim, vdim, dtype)
    if transposed:
        values = values.transpose(2, 3).contiguous()
    cu, seq, _ = _step(lengths, [0, 1, 2])
    n = H * dim + G * dim + G * vdim
    rows = _rand(g, T, n + H)
    bias, qw, kw = _rand(g, n), _rand(g, H * dim), _rand(g, G * dim)
    inv_freq = torch.tensor([250000.0 ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32, device=DEV) if rot else None
    k1, v1, k2, v2 = keys.clone(), values.clone(), keys.clone(), values.clone()
    q1 = ops.softcap_prepare(rows, bias, H, G, dim, vdim, qw, kw, 1e-6, inv_freq, positions, seq, dtype, table, k1, v1,
                             values_transposed=transposed)
    q2 = twin.softcap_prepare(rows, bias, H, G, dim, vdim, qw, kw, 1e-6, inv_freq, positions, seq, dtype, table, k2, v2,
                              values_transposed=transposed)
    _close(q1, q2, _tol(dtype))
    _close(k1, k2, _tol(dtype))
    _close(v1, v2, _tol(dtype))
    gate = rows[:, n:]
    for cap, window in ((0.0, 0), (5.0, 0), (50.0, 20), (2.0, 1)):
        got = ops.softcap_attention(q2, k2, v2, table, cu, kv_lens, seq, positions, max(lengths), int(kv_lens.max()),
                                    dim ** -0.5, cap, window=window, gate=gate, values_transposed=transposed,
                                    min_q_len=min(lengths))
        want = twin.softcap_attention(q2, k2, v2, table, cu, kv_lens, seq, positions, max(lengths), int(kv_lens.max()),
                                      dim ** -0.5, cap, window=window, gate=gate, values_transposed=transposed)
        _close(got, want, _tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim,vdim,transposed", [(32, 48, False), (64, 64, True)])
def test_one_far_key_carries_the_softmax(dtype, dim, vdim, transposed):
    """A query that matches one key hundreds of positions back, at a page's first or last place:
    with that key's score standing out the result is that key's value, and a kernel that skipped
    the key, its page or its tile would return something else. Once through the general kernel,
    once (bfloat16, equal sizes of 64, transposed values) through the matrix-core ones."""
    g = _gen(5)
    H = G = 2
    page, L = 16, 700
    keys, values, table, _, _ = _paged(g, [L - 1], [1], page, G, dim, vdim, dtype)
    if transposed:
        values = values.transpose(2, 3).contiguous()
    value_at = (lambda pg, off: values[pg, :, :, off]) if transposed else (lambda pg, off: values[pg, :, off])
    kw = dict(values_transposed=transposed)
    q = _rand(g, 1, H, dim, dtype=dtype)
    cu, seq, _ = _step([1], [0])
    positions = torch.tensor([L - 1], dtype=torch.int32, device=DEV)
    kv_lens = torch.tensor([L], dtype=torch.int32, device=DEV)
    for far in (0, 15, 16, 63, 64, 511, 512, L - 2, L - 1):
        k = keys.clone()
        pg = int(table[0, far // page])
        for h in range(G):
            k[pg, h, far % page] = (q[0, h].float() * 4.0).to(dtype)
        got = ops.softcap_attention(q, k, values, table, cu, kv_lens, seq, positions, 1, L, 1.0, 0.0, **kw)
        want = value_at(pg, far % page).float().reshape(1, -1)
        assert float((got.float() - want).abs().max()) < 0.05, far
        capped = ops.softcap_attention(q, k, values, table, cu, kv_lens, seq, positions, 1, L, 1.0, 500.0, **kw)
        assert float((capped.float() - want).abs().max()) < 0.05, far
        seen = ops.softcap_attention(q, k, values, table, cu, kv_lens, seq, positions, 1, L, 1.0, 0.0, window=L - 1 - far + 1, **kw)
        assert float((seen.float() - want).abs().max()) < 0.05, far
        if far < L - 1:
            hidden = ops.softcap_attention(q, k, values, table, cu, kv_lens, seq, positions, 1, L, 1.0, 0.0, window=L - 1 - far, **kw)
            assert float((hidden.float() - want).abs().max()) > 0.3, far


@pytest.mark.parametrize("dtype", DTYPES)
def test_scaled_sum(dtype):
    g = _gen(1)
    a, b = _rand(g, 9, 33, dtype=dtype), _rand(g, 9, 33, dtype=dtype)
    _close(ops.scaled_sum(a, 0.6, b, -1.1), twin.scaled_sum(a, 0.6, b, -1.1), _tol(dtype))
