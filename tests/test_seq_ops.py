"""The sequence-state ops one by one, on inputs made so that a fault shows:
a single far key that must win the softmax, keys on both sides of a page
border, the sink deciding a row, a state slot that is reused, a decay of 1.
Each op is compared with a few lines of plain per-row arithmetic written
here (no code of arks_amd); CPU cases run the reference ops, gpu-marked
cases the HIP kernels."""

import math

import pytest
import torch

from arks_amd import ops

DEVICES = [pytest.param("cpu", torch.float32, id="cpu-f32"),
           pytest.param("cuda", torch.float32, id="gpu-f32", marks=pytest.mark.gpu),
           pytest.param("cuda", torch.bfloat16, id="gpu-bf16", marks=pytest.mark.gpu)]


def i32(x, dev):
    return torch.tensor(x, dtype=torch.int32, device=dev)


def paged_cache(K, Vv, block_size, order, nblocks, dtype, dev):
    """Scatter K [L,G,D], V [L,G,V] into pages in the given page order."""
    L, G, D = K.shape
    kc = torch.zeros(nblocks, G, block_size, D, dtype=dtype, device=dev)
    vc = torch.zeros(nblocks, G, block_size, Vv.shape[2], dtype=dtype, device=dev)
    for j in range(L):
        kc[order[j // block_size], :, j % block_size] = K[j].to(dtype)
        vc[order[j // block_size], :, j % block_size] = Vv[j].to(dtype)
    return kc, vc


@pytest.mark.parametrize("dev,dtype", DEVICES)
@pytest.mark.parametrize("D", [16, 64])
@pytest.mark.parametrize("far", [0, 15, 16, 17, 250])
def test_one_far_key_wins_the_softmax(dev, dtype, D, far):
    """The last query matches exactly one key (first token, either side of
    a page border, hundreds back): the output must be that key's value."""
    torch.manual_seed(far)
    L, G, H, bs = 300, 1, 2, 16
    K = torch.randn(L, G, D) * 0.05
    Vv = torch.randn(L, G, D)
    e = torch.zeros(D)
    e[3] = 1.0
    K[far, 0] = 6.0 * e
    order = torch.randperm(40).tolist()
    kc, vc = paged_cache(K, Vv, bs, order, 40, dtype, dev)
    for n_new in (1, 5):  # decoded alone, and as the last row of a portion
        q = torch.randn(n_new, H, D) * 0.05
        q[-1, :] = 6.0 * e
        qd = q.to(dtype).to(dev)
        tiles = (ops.sink_attention_tiles([n_new], [L], H, G, D, dev)
                 if dev == "cuda" else None)
        out = ops.attention_sink_paged(
            qd, kc, vc, i32([order[:19]], dev), i32([L], dev), i32([0, n_new], dev),
            i32([0] * n_new, dev), 1.0, sink=True, inv_freq_v=None,
            max_q_len=n_new, positions=torch.arange(L - n_new, L, device=dev),
            tiles=tiles)
        got = out[-1].float().cpu()
        # e^36 against 300 keys near e^0 and the sink's e^0
        assert torch.allclose(got, Vv[far, 0].expand(H, D).to(dtype).float(),
                              atol=3e-2 if dtype == torch.bfloat16 else 1e-4), (n_new, far)


@pytest.mark.parametrize("dev,dtype", DEVICES)
@pytest.mark.parametrize("D", [16, 64])
def test_sink_takes_its_share(dev, dtype, D):
    """All scores 0: n keys and the sink share the weight, so the output is
    sum(v) / (n + 1), not the mean; very negative scores give 0."""
    L, G, H, bs = 37, 1, 1, 16
    Vv = torch.randn(L, G, D)
    kc, vc = paged_cache(torch.zeros(L, G, D), Vv, bs, [2, 0, 1], 3, dtype, dev)
    q = torch.zeros(1, H, D, dtype=dtype, device=dev)
    args = (kc, vc, i32([[2, 0, 1]], dev), i32([L], dev), i32([0, 1], dev), i32([0], dev))
    tiles = ops.sink_attention_tiles([1], [L], H, G, D, dev) if dev == "cuda" else None
    kw = dict(inv_freq_v=None, max_q_len=1, positions=torch.tensor([L - 1], device=dev),
              tiles=tiles)
    out = ops.attention_sink_paged(q, *args, 1.0, sink=True, **kw)
    want = Vv[:, 0].to(dtype).float().sum(0) / (L + 1)
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-5
    assert torch.allclose(out[0, 0].float().cpu(), want, atol=tol)
    out = ops.attention_sink_paged(q, *args, 1.0, sink=False, **kw)
    assert torch.allclose(out[0, 0].float().cpu(), want * (L + 1) / L, atol=tol)
    kc2, _ = paged_cache(torch.full((L, G, D), -4.0), Vv, bs, [2, 0, 1], 3, dtype, dev)
    q1 = torch.ones(1, H, D, dtype=dtype, device=dev)
    out = ops.attention_sink_paged(q1, kc2, *args[1:], 1.0, sink=True, **kw)
    assert out.float().abs().max() < 1e-6 * math.exp(30)  # e^(-4D) << 1
    assert out.float().abs().max() < 1e-3


@pytest.mark.parametrize("dev,dtype", DEVICES)
def test_rotated_values_come_back_in_the_query_frame(dev, dtype):
    """One key at position j holds value v turned by j; a query at position i
    that sees only it (strongly) must return v turned by j - i."""
    D, bs = 8, 16
    inv = torch.tensor([1.0, 0.5, 0.1, 0.01])
    j, i = 5, 21
    v = torch.randn(D)
    k = torch.zeros(i + 1, 1, D)
    k[j, 0, 0] = 8.0
    vals = torch.zeros(i + 1, 1, D)
    kc, vc = paged_cache(k, vals, bs, [1, 0], 2, dtype, dev)
    # store v through the op that fills the cache (rotation by the position)
    qkv_q = torch.zeros(1, 1, D, dtype=dtype, device=dev)
    ops.qk_norm_rope_cache(
        qkv_q, k[j:j + 1].to(dtype).to(dev), v.view(1, 1, D).to(dtype).to(dev), None, None,
        1e-5, torch.tensor([j], device=dev), torch.zeros(0, device=dev),
        inv.to(dev), kc, vc, torch.tensor([1 * bs + j], device=dev))
    q = torch.zeros(1, 1, D, dtype=dtype, device=dev)
    q[0, 0, 0] = 8.0
    out = ops.attention_sink_paged(
        q, kc, vc, i32([[1, 0]], dev), i32([i + 1], dev), i32([0, 1], dev), i32([0], dev),
        1.0, sink=True, inv_freq_v=inv.to(dev), max_q_len=1,
        positions=torch.tensor([i], device=dev))
    ang = (j - i) * inv
    want = torch.empty(D)
    want[0::2] = v[0::2] * torch.cos(ang) - v[1::2] * torch.sin(ang)
    want[1::2] = v[1::2] * torch.cos(ang) + v[0::2] * torch.sin(ang)
    assert torch.allclose(out[0, 0].float().cpu(), want,
                          atol=5e-2 if dtype == torch.bfloat16 else 1e-4)


@pytest.mark.parametrize("dev,dtype", DEVICES)
def test_lightning_keeps_a_far_token_with_decay_one_and_forgets_with_small(dev, dtype):
    H, D, V, T = 2, 8, 8, 200
    q = torch.zeros(T, H, D)
    k = torch.zeros(T, H, D)
    v = torch.zeros(T, H, V)
    k[0, :, 1] = 5.0   # silu(5) ~ 4.97
    v[0, :, 2] = 5.0
    q[T - 1, :, 1] = 5.0
    decay = torch.tensor([1.0, 0.5])
    state = torch.zeros(3, H, D, V, device=dev)
    s5 = 5.0 / (1 + math.exp(-5.0))
    # whole, and cut in portions through a reused slot holding garbage
    for cuts in ([T], [1, 2, 64, 33, 100]):
        state.fill_(7.0)
        at, o_last = 0, None
        for n in cuts:
            o = ops.lightning_scan(
                q[at:at + n].to(dtype).to(dev), k[at:at + n].to(dtype).to(dev),
                v[at:at + n].to(dtype).to(dev), decay.to(dev), state,
                i32([0, n], dev), i32([at + n], dev), i32([1], dev), max_q_len=n)
            at += n
            o_last = o[-1].cpu()
        assert abs(float(o_last[0, 2]) - s5 ** 3) < 0.05 * s5 ** 3
        assert abs(float(o_last[1, 2])) < 1e-20
        assert float(state[0].min()) == 7.0 and float(state[2].min()) == 7.0


@pytest.mark.parametrize("dev,dtype", DEVICES)
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_conv_history_across_portions_of_one_and_two(dev, dtype, taps):
    C, T = 5, 9
    x = torch.randn(T, C)
    w = torch.randn(C, taps)
    b = torch.randn(C)
    xd = x.to(dtype).float()
    want = torch.zeros(T, C)
    for t in range(T):
        acc = b.clone()
        for j in range(taps):
            s = t - (taps - 1 - j)
            if s >= 0:
                acc += w[:, j] * xd[s]
        want[t] = acc * torch.sigmoid(acc)
    state = (torch.full((2, taps - 1, C), 9.0, device=dev) if taps > 1 else None)
    outs, at = [], 0
    for n in (1, 1, 2, 1, 4):
        outs.append(ops.causal_conv_silu(
            x[at:at + n].to(dtype).to(dev), w.to(dev), b.to(dev), state,
            i32([0, n], dev), i32([at + n], dev), i32([1], dev), i32([0] * n, dev)))
        at += n
    got = torch.cat(outs).float().cpu()
    assert torch.allclose(got, want, atol=5e-2 if dtype == torch.bfloat16 else 1e-5)


@pytest.mark.parametrize("dev,dtype", DEVICES)
def test_token_shift_first_row_and_padding_rows(dev, dtype):
    W = 6
    x = torch.randn(5, W, device=dev)
    w = torch.rand(W, device=dev)
    state = torch.full((2, W), 3.0, device=dev)
    # seq 0: 3 rows starting at position 0 (slot 1); seq 1: one row at
    # position 4 (slot 0, reads the stored row); seq 2: padding row
    xs, xa = ops.token_shift(x, w, state, i32([0, 3, 4, 5], dev), i32([3, 5, 1], dev),
                             i32([1, 0, -1], dev), i32([0, 0, 0, 1, 2], dev), dtype)
    xc = x.cpu()
    wc = w.cpu()
    want = torch.stack([
        xc[0] * (1 - wc), xc[1] + (xc[0] - xc[1]) * wc, xc[2] + (xc[1] - xc[2]) * wc,
        xc[3] + (3.0 - xc[3]) * wc, xc[4] * (1 - wc)])
    tol = 3e-2 if dtype == torch.bfloat16 else 1e-6
    assert torch.allclose(xs.float().cpu(), want, atol=tol)
    assert torch.allclose(xa.float().cpu(), xc, atol=tol)
    assert torch.equal(state[1].cpu(), xc[2]) and torch.equal(state[0].cpu(), xc[3])


@pytest.mark.parametrize("dev,dtype", DEVICES)
def test_selective_scan_remembers_through_a_slow_channel(dev, dtype):
    """Channel 0 decays slowly (A ~ 0), channel 1 fast: an input at the first
    token is still read out 150 tokens later on channel 0 only."""
    C, N, R, T = 2, 4, 1, 151
    u = torch.zeros(T, C)
    u[0] = 2.0
    dbc = torch.zeros(T, R + 2 * N)
    dbc[:, R:R + N] = 1.0       # B
    dbc[:, R + N:] = 1.0        # C
    z = torch.full((T, C), 20.0)  # silu(20) ~ 20
    dt_w = torch.zeros(C, R)
    dt_b = torch.zeros(C)       # dt = softplus(0) = ln 2
    A = torch.tensor([[-1e-4] * N, [-3.0] * N])
    Dp = torch.zeros(C)
    ln2 = math.log(2.0)
    want0 = N * ln2 * 2.0 * math.exp(-1e-4 * ln2 * (T - 1)) * 20.0
    state = torch.full((2, C, N), 5.0, device=dev)
    for cuts in ([T], [2, 1, 100, 48]):
        at = 0
        for n in cuts:
            y = ops.selective_scan(
                u[at:at + n].to(dtype).to(dev), dbc[at:at + n].to(dtype).to(dev),
                z[at:at + n].to(dtype).to(dev), dt_w.to(dev), dt_b.to(dev), A.to(dev),
                Dp.to(dev), state, i32([0, n], dev), i32([at + n], dev), i32([0], dev),
                max_q_len=n)
            at += n
        last = y[-1].float().cpu()
        assert abs(float(last[0]) - want0) < 0.02 * want0
        assert abs(float(last[1])) < 1e-6
        assert float(state[1].min()) == 5.0


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("lens", [[65], [64, 1, 200], [129, 128, 63]])
def test_chunk_parallel_scans_equal_row_by_row(dtype, lens):
    """The chunk-parallel prefill of both recurrent mixers against the same
    kernels walking every row in order, with old state in the slots."""
    dev = "cuda"
    torch.manual_seed(sum(lens))
    T, S = sum(lens), len(lens)
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    starts = [0, 7, 300][:S]
    seq_lens = [s + n for s, n in zip(starts, lens)]
    slots = [2, 0, 3][:S]
    meta = (i32(cu, dev), i32(seq_lens, dev), i32(slots, dev))
    chunks = ops.scan_chunks(lens, torch.device(dev))
    # lightning
    H, D, V = 3, 16, 24
    q, k, v = (torch.randn(T, H, n, device=dev).to(dtype) for n in (D, D, V))
    decay = torch.tensor([1.0, 0.97, 0.6], device=dev)
    st0 = torch.randn(4, H, D, V, device=dev)
    sa, sb = st0.clone(), st0.clone()
    a = ops.lightning_scan(q, k, v, decay, sa, *meta, max_q_len=max(lens))
    b = ops.lightning_scan(q, k, v, decay, sb, *meta, max_q_len=max(lens), chunks=chunks)
    assert torch.allclose(a, b, rtol=1e-4, atol=1e-4)
    assert torch.allclose(sa, sb, rtol=1e-4, atol=1e-4)
    # selective scan, with dt from a GEMM and projected in the kernel
    C, N, R = 40, 12, 5
    u = torch.randn(T, C, device=dev).to(dtype)
    dbc = torch.randn(T, R + 2 * N, device=dev).to(dtype)
    z = torch.randn(T, C, device=dev).to(dtype)
    dt_w = torch.randn(C, R, device=dev) * 0.3
    dt_b = torch.randn(C, device=dev) - 1.0
    A = -torch.rand(C, N, device=dev) * 2
    Dp = torch.randn(C, device=dev)
    st0 = torch.randn(4, C, N, device=dev)
    dt_pre = dbc[:, :R].float() @ dt_w.t()
    outs = []
    for kw in ({}, {"chunks": chunks}, {"dt_pre": dt_pre, "chunks": chunks}):
        st = st0.clone()
        y = ops.selective_scan(u, dbc, z, dt_w, dt_b, A, Dp, st, *meta,
                               max_q_len=max(lens), **kw)
        outs.append((y.float(), st))
    tol = 2e-2 if dtype == torch.bfloat16 else 2e-4
    for y, st in outs[1:]:
        assert torch.allclose(y, outs[0][0], rtol=tol, atol=tol)
        assert torch.allclose(st, outs[0][1], rtol=1e-4, atol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("D,V", [(32, 32), (64, 64), (64, 128), (128, 64), (128, 128)])
def test_lightning_matrix_core_prefill_equals_general_kernel(D, V):
    """bf16 rows, head sizes the matrix-core kernels are built for: chunk
    ends of 1, 63, 64 and 65 rows, decays 1, 0 and in between, old state."""
    dev = "cuda"
    torch.manual_seed(D + V)
    lens = [65, 129, 200, 64]
    T, H = sum(lens), 4
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    starts = [0, 9, 500, 0]
    meta = (i32(cu, dev), i32([s + n for s, n in zip(starts, lens)], dev),
            i32([1, 3, 0, 2], dev))
    chunks = ops.scan_chunks(lens, torch.device(dev))
    q, k, v = (torch.randn(T, H, n, device=dev).to(torch.bfloat16) for n in (D, D, V))
    decay = torch.tensor([1.0, 0.0, 0.9, 0.999], device=dev)
    st0 = torch.randn(4, H, D, V, device=dev)
    res = {}
    for flag in (False, True):
        ops.use_lightning_mfma = flag
        try:
            st = st0.clone()
            o = ops.lightning_scan(q, k, v, decay, st, *meta, max_q_len=max(lens),
                                   chunks=chunks)
        finally:
            ops.use_lightning_mfma = True
        res[flag] = (o, st)
    scale = res[False][0].abs().max()
    assert (res[True][0] - res[False][0]).abs().max() < 1e-2 * scale
    sscale = res[False][1].abs().max()
    assert (res[True][1] - res[False][1]).abs().max() < 1e-2 * sscale
