"""The one-kernel route of dc_decode_layer for short contexts (csrc/small.hip).

dc_decode_layer takes it when no dense scores are asked for, the ids may come in any order and
every block of the launch fits on the chip at once.  Checked against the oracle like the other
routes: ids bit-exact against ``oracle.topk_select`` of the GPU's dense scores (the kept set of
search_bruteforce, diffcache_cpu/src/nsw.rs:592-630, ties to the lower id), attention within
2e-3 of the float64 softmax over the oracle's row set (src/diffcache/base.py:134-142).
"""
import numpy as np
import pytest
import torch

from oracle import oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
hip = None


@pytest.fixture(scope="module", autouse=True)
def _load():
    global hip
    from diffcache_amd import _hip
    hip = _hip
    yield


def to_dev_bf16(u16):
    return torch.from_numpy(u16.view(np.int16).copy()).view(torch.bfloat16).to(DEV)


def to_np_u16(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bf16_close(got_f32, want_f64):
    tol = np.maximum(2e-3, np.abs(want_f64) * 2.0 ** -8)
    return bool(np.all(np.abs(got_f32 - want_f64) <= tol))


def run_case(k, v, q, nk, nv, n_ctx, budget, p, s, mode, reps=2, n_recent_dev=None, recent_cap=None, ws=None):
    """k, v (b, hkv, n_max, hd) u16; q (b, hq, hd); nk, nv (b, hkv, hd) or None.  Calls
    dc_decode_layer (no scores, ORDER_ANY) `reps` times on one workspace and checks every call."""
    b, hkv, n_max, hd = k.shape
    hq = q.shape[1]
    g = hq // hkv
    p_len, s_len, lo, hi = orc.region_split(n_ctx, p, s)
    region = hi - lo
    k_eff = min(budget, region)
    n_units = b * hkv
    kd, vd, qd = to_dev_bf16(k), to_dev_bf16(v), to_dev_bf16(q)
    nkd = None if nk is None else to_dev_bf16(nk)
    nvd = None if nv is None else to_dev_bf16(nv)
    cap = s_len if recent_cap is None else recent_cap
    if ws is None:
        ws = hip.alloc_workspace(hip.layer_workspace_bytes(n_units, region, budget, g, hd,
                                                           k_eff + p_len + cap + 1), DEV)
    dense = hip.score(kd, qd, lo, region, mode, q_group=g).cpu().numpy() if region > 0 else None
    lse = torch.empty((b, hq), dtype=torch.float32, device=DEV)
    for rep in range(reps):
        idx = torch.full((n_units, max(budget, 1)), -1, dtype=torch.int32, device=DEV)
        out = torch.full((b, hq, hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        args = (qd, kd, vd, p_len, hi, cap, budget, None, idx, out, ws, nkd, nvd)
        kw = dict(lse=lse, mode=mode, order=hip.ORDER_ANY, select_state_ready=rep > 0, n_recent_dev=n_recent_dev)
        hip.decode_layer(*args, **kw)
        hip.decode_layer_status(*args, **kw)        # waits for the stream; no bounded wait ran out
        ids = idx.cpu().numpy()[:, :k_eff].astype(np.int64)
        got = orc.bf16_to_f32(to_np_u16(out))
        got_lse = lse.cpu().numpy()
        for u in range(n_units):
            bi, h = divmod(u, hkv)
            want = orc.topk_select(dense[u], k_eff, mode).astype(np.int64) if k_eff else np.zeros(0, np.int64)
            assert np.array_equal(np.sort(ids[u]), np.sort(want)), (rep, u)
            rows = np.concatenate([want + lo, np.arange(p_len), np.arange(hi, hi + s_len)]).astype(np.int64)
            o, l = orc.sparse_attention(q[bi, h * g:(h + 1) * g], k[bi, h][rows], v[bi, h][rows],
                                        None if nk is None else nk[bi, h], None if nv is None else nv[bi, h])
            assert bf16_close(got[bi, h * g:(h + 1) * g], o), (rep, u)
            assert np.allclose(got_lse[bi, h * g:(h + 1) * g], l, rtol=1e-4, atol=1e-4), (rep, u)
    return ws


def rand_bf16(rng, *shape, scale=1.0):
    return orc.f32_to_bf16((rng.standard_normal(shape) * scale).astype(np.float32))


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("hd,hq,hkv", [(128, 8, 2), (64, 7, 7), (256, 16, 2), (128, 14, 2)])
def test_small_context_layer_matches_oracle(mode, hd, hq, hkv):
    rng = np.random.default_rng(300 + hd + hq)
    b, n_ctx = 2, 5000
    k, v = rand_bf16(rng, b, hkv, n_ctx + 3, hd), rand_bf16(rng, b, hkv, n_ctx + 3, hd)
    q = rand_bf16(rng, b, hq, hd)
    nk, nv = rand_bf16(rng, b, hkv, hd), rand_bf16(rng, b, hkv, hd)
    print(f"small context hd={hd} hq={hq} hkv={hkv} mode={mode}", flush=True)
    run_case(k, v, q, nk, nv, n_ctx, 300, 4, 64, mode)


def test_small_context_edge_sizes_share_one_workspace():
    """Regions of 1 row, fewer rows than the budget, no current token, no sinks; consecutive calls of
    different sizes each initialise their own state."""
    rng = np.random.default_rng(301)
    b, hq, hkv, hd = 1, 8, 2, 128
    for n_ctx, budget, p, s, tok in [(70, 64, 4, 64, True), (69, 64, 4, 64, True), (300, 512, 4, 64, False),
                                     (4000, 128, 0, 0, True), (2500, 1, 2, 3, True), (9000, 4096, 4, 64, True)]:
        print(f"small context n_ctx={n_ctx} budget={budget} p={p} s={s} tok={tok}", flush=True)
        k, v = rand_bf16(rng, b, hkv, n_ctx, hd), rand_bf16(rng, b, hkv, n_ctx, hd)
        q = rand_bf16(rng, b, hq, hd)
        nk = rand_bf16(rng, b, hkv, hd) if tok else None
        nv = rand_bf16(rng, b, hkv, hd) if tok else None
        run_case(k, v, q, nk, nv, n_ctx, budget, p, s, orc.MODE_REF_DIST)


@pytest.mark.parametrize("mode", [0, 1])
def test_small_context_ties(mode):
    """Integer-valued keys: scores tie in large groups, the boundary goes to the lower ids.  A zero
    query makes every row tie (more candidates than a block ranks in LDS: the radix-select path)."""
    rng = np.random.default_rng(302 + mode)
    b, hq, hkv, hd, n_ctx = 1, 12, 3, 128, 20000
    k = orc.f32_to_bf16(rng.integers(-2, 3, (b, hkv, n_ctx, hd)).astype(np.float32))
    v = rand_bf16(rng, b, hkv, n_ctx, hd)
    q = orc.f32_to_bf16(rng.integers(-1, 2, (b, hq, hd)).astype(np.float32))
    q[0, 8:12] = 0                                      # unit 2: everything ties, lowest ids win
    k[0, 1, 5000:15000] = k[0, 1, 4999]                 # unit 1: ten thousand identical rows
    nk, nv = rand_bf16(rng, b, hkv, hd), rand_bf16(rng, b, hkv, hd)
    run_case(k, v, q, nk, nv, n_ctx, 1500, 4, 64, mode)


def test_small_context_benchmark_shape_with_a_device_side_window():
    """Benchmark configuration 2 (8 units x 32700 rows, k 1024, outlier channels); the recent
    window's length is read from the device and grows between the calls."""
    rng = np.random.default_rng(303)
    b, hq, hkv, hd, n0, cap = 1, 32, 8, 128, 32768, 72
    scale = np.exp(rng.standard_normal((1, hkv, 1, hd))).astype(np.float32)
    k = orc.f32_to_bf16(rng.standard_normal((b, hkv, n0 + 8, hd)).astype(np.float32) * scale)
    v = rand_bf16(rng, b, hkv, n0 + 8, hd)
    q = rand_bf16(rng, b, hq, hd)
    nk, nv = rand_bf16(rng, b, hkv, hd), rand_bf16(rng, b, hkv, hd)
    counter = torch.zeros((1,), dtype=torch.int32, device=DEV)
    ws = None
    for step in range(3):
        # the region stays [4, n0 - 64); the window holds 64 + step rows of its capacity of 72
        counter.fill_(64 + step)
        n_ctx = n0 + step
        # oracle side: prefix 4, suffix 64 + step  ->  same region; the store holds the whole window
        ws = run_case(k, v, q, nk, nv, n_ctx, 1024, 4, 64 + step,
                      orc.MODE_REF_DIST, reps=1, n_recent_dev=counter, recent_cap=cap, ws=ws)


def test_small_context_bounded_wait_is_reported():
    """With a wait limit of one poll the blocks give up their waits.  The kernel still ends; the
    step cannot pass for a good one (NaN outputs, ids 0xffffffff); the host learns of it without
    a synchronising call (dc_decode_layer_errors); later calls on the workspace return NaN as long
    as the state is not initialised again; and the library initialises it again by itself on the
    next call, although that call says select_state_ready."""
    rng = np.random.default_rng(304)
    b, hq, hkv, hd, n_ctx = 1, 8, 2, 128, 30000
    k, v = rand_bf16(rng, b, hkv, n_ctx, hd), rand_bf16(rng, b, hkv, n_ctx, hd)
    q = rand_bf16(rng, b, hq, hd)
    kd, vd, qd = to_dev_bf16(k), to_dev_bf16(v), to_dev_bf16(q)
    p_len, s_len, lo, hi = orc.region_split(n_ctx, 4, 64)
    ws = hip.alloc_workspace(hip.layer_workspace_bytes(b * hkv, hi - lo, 512, hq // hkv, hd, 512 + 4 + 64 + 1), DEV)
    idx = torch.zeros((b * hkv, 512), dtype=torch.int32, device=DEV)
    out = torch.zeros((b, hq, hd), dtype=torch.bfloat16, device=DEV)
    lse = torch.zeros((b, hq), dtype=torch.float32, device=DEV)
    args = (qd, kd, vd, p_len, hi, s_len, 512, None, idx, out, ws)
    errors0 = hip.decode_layer_errors()
    hip.lib.dc_set_wait_limit(1)
    try:
        print("forced give-up: one-kernel launch with a wait limit of one poll", flush=True)
        hip.decode_layer(*args, lse=lse, order=hip.ORDER_ANY)
        assert hip.last_route() == hip.ROUTE_ONE_KERNEL
        with pytest.raises(hip.DiffCacheError, match="bounded wait"):
            hip.decode_layer_status(*args, order=hip.ORDER_ANY)
    finally:
        hip.lib.dc_set_wait_limit(0)
    bad_units = [u for u in range(b * hkv) if (idx[u] == -1).all()]
    assert bad_units, "no unit reported its failure in the ids"
    g = hq // hkv
    for u in bad_units:
        assert torch.isnan(out.view(b * hkv, g, hd)[u].float()).all()
        assert torch.isnan(lse.view(b * hkv, g)[u]).all()
    for u in range(b * hkv):        # a unit is either marked as a whole or not at all in its output
        o = torch.isnan(out.view(b * hkv, g, hd)[u].float())
        assert o.all() or not o.any()
    assert hip.decode_layer_errors() > errors0              # read from pinned host memory, no stream wait
    # with the default limit again, on a second workspace nothing is wrong
    run_case(k, v, q, None, None, n_ctx, 512, 4, 64, orc.MODE_REF_DIST, reps=2)
    # the workspace of the failed call: the caller still says "ready"; the library knows better
    print("forced give-up: next call on the same workspace, select_state_ready=1", flush=True)
    idx.fill_(7)
    out.zero_()
    hip.decode_layer(*args, order=hip.ORDER_ANY, select_state_ready=True)
    assert hip.last_route() == hip.ROUTE_ONE_KERNEL
    hip.decode_layer_status(*args, order=hip.ORDER_ANY)     # the error words are clear again
    assert not torch.isnan(out.float()).any()
    dense = hip.score(kd, qd, lo, hi - lo, orc.MODE_REF_DIST, q_group=g).cpu().numpy()
    ids = idx.cpu().numpy().astype(np.int64)
    for u in range(b * hkv):
        want = orc.topk_select(dense[u], 512, orc.MODE_REF_DIST).astype(np.int64)
        assert np.array_equal(np.sort(ids[u]), np.sort(want)), u
    run_case(k, v, q, None, None, n_ctx, 512, 4, 64, orc.MODE_REF_DIST, reps=2, ws=ws)


def test_small_context_sticky_error_marks_later_calls_until_initialised():
    """A captured graph cannot be mended by the library (its launches are fixed).  What it must
    not do is return stale numbers: with the unit's error word set, every later one-kernel launch
    on the workspace marks its outputs, until the state is initialised again."""
    rng = np.random.default_rng(307)
    b, hq, hkv, hd, n_ctx = 1, 8, 2, 128, 9000
    k, v, q = rand_bf16(rng, b, hkv, n_ctx, hd), rand_bf16(rng, b, hkv, n_ctx, hd), rand_bf16(rng, b, hq, hd)
    kd, vd, qd = to_dev_bf16(k), to_dev_bf16(v), to_dev_bf16(q)
    p_len, s_len, lo, hi = orc.region_split(n_ctx, 4, 64)
    ws = hip.alloc_workspace(hip.layer_workspace_bytes(b * hkv, hi - lo, 256, hq // hkv, hd, 256 + 69), DEV)
    idx = torch.zeros((b * hkv, 256), dtype=torch.int32, device=DEV)
    out = torch.zeros((b, hq, hd), dtype=torch.bfloat16, device=DEV)
    args = (qd, kd, vd, p_len, hi, s_len, 256, None, idx, out, ws)
    # two calls enqueued back to back, the second before the host can have seen the first fail
    hip.lib.dc_set_wait_limit(1)
    try:
        print("sticky error: failing launch, then a launch enqueued behind it", flush=True)
        hip.decode_layer(*args, order=hip.ORDER_ANY)
    finally:
        hip.lib.dc_set_wait_limit(0)
    out2 = torch.zeros_like(out)
    idx2 = torch.zeros_like(idx)
    args2 = (qd, kd, vd, p_len, hi, s_len, 256, None, idx2, out2, ws)
    # (the error count is not asked in between: nothing on the host has looked at the mailbox yet
    #  unless this call does, in which case it initialises the state and the result is good)
    hip.decode_layer(*args2, order=hip.ORDER_ANY, select_state_ready=True)
    torch.cuda.synchronize()
    first_bad = torch.isnan(out.float()).any().item()
    assert first_bad
    healed = not torch.isnan(out2.float()).any().item()
    if healed:      # the host saw the failure in time: the second call must then be right
        dense = hip.score(kd, qd, lo, hi - lo, orc.MODE_REF_DIST, q_group=hq // hkv).cpu().numpy()
        for u in range(b * hkv):
            want = orc.topk_select(dense[u], 256, orc.MODE_REF_DIST).astype(np.int64)
            assert np.array_equal(np.sort(idx2[u].cpu().numpy().astype(np.int64)), np.sort(want)), u
    else:           # it did not: every unit whose error word was set is marked, none is stale
        g = hq // hkv
        for u in range(b * hkv):
            if torch.isnan(out.view(b * hkv, g, hd)[u].float()).any():
                assert torch.isnan(out2.view(b * hkv, g, hd)[u].float()).all(), u
                assert (idx2[u] == -1).all(), u
    run_case(k, v, q, None, None, n_ctx, 256, 4, 64, orc.MODE_REF_DIST, reps=2, ws=ws)


def test_two_streams_never_run_the_one_kernel_route_side_by_side():
    """Two sequences decoded on two streams of one process.  While the one-kernel launch of the
    first is still in flight, a call on the second stream takes the kernel chain (two launches of
    the kernel would starve each other of CUs); both calls are right.  Once the first has ended,
    the second stream gets the kernel again."""
    rng = np.random.default_rng(308)
    b, hq, hkv, hd, n_ctx, budget = 1, 8, 2, 128, 20000, 384
    g = hq // hkv
    p_len, s_len, lo, hi = orc.region_split(n_ctx, 4, 64)
    seqs = []
    for _ in range(2):
        k, v, q = rand_bf16(rng, b, hkv, n_ctx, hd), rand_bf16(rng, b, hkv, n_ctx, hd), rand_bf16(rng, b, hq, hd)
        kd, vd, qd = to_dev_bf16(k), to_dev_bf16(v), to_dev_bf16(q)
        sk = hip.Sketch(kd).build(kd, lo, hi - lo)
        ws = hip.alloc_workspace(hip.layer_workspace_bytes(b * hkv, hi - lo, budget, g, hd, budget + 69), DEV)
        idx = torch.zeros((b * hkv, budget), dtype=torch.int32, device=DEV)
        out = torch.zeros((b, hq, hd), dtype=torch.bfloat16, device=DEV)
        seqs.append(dict(k=k, v=v, q=q, kd=kd, vd=vd, qd=qd, sk=sk, ws=ws, idx=idx, out=out))
    torch.cuda.synchronize()
    s_a, s_b = torch.cuda.Stream(), torch.cuda.Stream()
    big = torch.randn((8192, 8192), device=DEV, dtype=torch.bfloat16)
    big = (big @ big).clamp_(-1, 1)         # (the GEMM library loads its kernels on first use)
    torch.cuda.synchronize()
    routes = []

    def call(sq, sketch):
        hip.decode_layer(sq["qd"], sq["kd"], sq["vd"], p_len, hi, s_len, budget, None, sq["idx"], sq["out"],
                         sq["ws"], order=hip.ORDER_ANY, sketch=sq["sk"] if sketch else None)
        routes.append(hip.last_route())

    print("two streams: stream A busy, one-kernel launch queued behind it; stream B calls meanwhile", flush=True)
    with torch.cuda.stream(s_a):
        for _ in range(40):                 # tens of milliseconds of work in front of A's call
            big = (big @ big).clamp_(-1, 1)
        call(seqs[0], sketch=True)
    with torch.cuda.stream(s_b):
        call(seqs[1], sketch=True)          # A's kernel has not even started: B must not launch a second one
        call(seqs[1], sketch=False)         # still pending
    torch.cuda.synchronize()
    assert routes == [hip.ROUTE_ONE_KERNEL, hip.ROUTE_SKETCH, hip.ROUTE_STREAM], routes
    with torch.cuda.stream(s_b):
        call(seqs[1], sketch=True)          # nothing of A is in flight any more
    torch.cuda.synchronize()
    assert routes[-1] == hip.ROUTE_ONE_KERNEL
    for sq in seqs:
        dense = hip.score(sq["kd"], sq["qd"], lo, hi - lo, orc.MODE_REF_DIST, q_group=g).cpu().numpy()
        ids = sq["idx"].cpu().numpy().astype(np.int64)
        got = orc.bf16_to_f32(to_np_u16(sq["out"]))
        for u in range(b * hkv):
            bi, h = divmod(u, hkv)
            want = orc.topk_select(dense[u], budget, orc.MODE_REF_DIST).astype(np.int64)
            assert np.array_equal(np.sort(ids[u]), np.sort(want)), u
            rows = np.concatenate([want + lo, np.arange(p_len), np.arange(hi, hi + s_len)]).astype(np.int64)
            o, _ = orc.sparse_attention(sq["q"][bi, h * g:(h + 1) * g], sq["k"][bi, h][rows], sq["v"][bi, h][rows],
                                        None, None)
            assert bf16_close(got[bi, h * g:(h + 1) * g], o), u


def test_one_kernel_route_under_capture_needs_the_callers_word():
    """A stream under capture: the call takes the kernel chain unless the caller vouches for an
    exclusive GPU (ONE_KERNEL_EXCLUSIVE); replays of both graphs equal the eager result, with eager
    work and synchronisation between the replays."""
    rng = np.random.default_rng(309)
    b, hq, hkv, hd, n_ctx, budget = 1, 8, 2, 128, 12000, 256
    g = hq // hkv
    p_len, s_len, lo, hi = orc.region_split(n_ctx, 4, 64)
    k, v = rand_bf16(rng, b, hkv, n_ctx, hd), rand_bf16(rng, b, hkv, n_ctx, hd)
    kd, vd = to_dev_bf16(k), to_dev_bf16(v)
    qd = to_dev_bf16(rand_bf16(rng, b, hq, hd))
    res = {}
    for policy in (hip.ONE_KERNEL_AUTO, hip.ONE_KERNEL_EXCLUSIVE):
        ws = hip.alloc_workspace(hip.layer_workspace_bytes(b * hkv, hi - lo, budget, g, hd, budget + 69), DEV)
        idx = torch.zeros((b * hkv, budget), dtype=torch.int32, device=DEV)
        out = torch.zeros((b, hq, hd), dtype=torch.bfloat16, device=DEV)
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):       # every kernel once outside capture; leaves the state ready
            hip.decode_layer(qd, kd, vd, p_len, hi, s_len, budget, None, idx, out, ws, order=hip.ORDER_ANY,
                             one_kernel=policy)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            hip.decode_layer(qd, kd, vd, p_len, hi, s_len, budget, None, idx, out, ws, order=hip.ORDER_ANY,
                             select_state_ready=True, one_kernel=policy)
            route = hip.last_route()
        assert route == (hip.ROUTE_ONE_KERNEL if policy == hip.ONE_KERNEL_EXCLUSIVE else hip.ROUTE_STREAM)
        res[policy] = (graph, idx, out, ws)
    for rep in range(3):
        qd.copy_(to_dev_bf16(rand_bf16(rng, b, hq, hd)))
        idx_e = torch.zeros((b * hkv, budget), dtype=torch.int32, device=DEV)
        out_e = torch.zeros((b, hq, hd), dtype=torch.bfloat16, device=DEV)
        ws_e = hip.alloc_workspace(hip.layer_workspace_bytes(b * hkv, hi - lo, budget, g, hd, budget + 69), DEV)
        hip.decode_layer(qd, kd, vd, p_len, hi, s_len, budget, None, idx_e, out_e, ws_e, order=hip.ORDER_ANY,
                         one_kernel=hip.ONE_KERNEL_NEVER)
        torch.cuda.synchronize()
        for policy, (graph, idx, out, ws) in res.items():
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(torch.sort(idx, dim=1).values, torch.sort(idx_e, dim=1).values), (rep, policy)
            assert torch.allclose(out.float(), out_e.float(), atol=4e-3, rtol=2.0 ** -6), (rep, policy)


def test_prepared_layer_call_equals_decode_layer():
    """hip.LayerCall builds the argument struct once; calling it equals decode_layer."""
    rng = np.random.default_rng(305)
    b, hq, hkv, hd, n_ctx, budget = 1, 8, 2, 128, 20000, 256
    k, v, q = rand_bf16(rng, b, hkv, n_ctx, hd), rand_bf16(rng, b, hkv, n_ctx, hd), rand_bf16(rng, b, hq, hd)
    kd, vd, qd = to_dev_bf16(k), to_dev_bf16(v), to_dev_bf16(q)
    p_len, s_len, lo, hi = orc.region_split(n_ctx, 4, 64)
    ws = hip.alloc_workspace(hip.layer_workspace_bytes(b * hkv, hi - lo, budget, hq // hkv, hd, budget + 69), DEV)
    for order in (hip.ORDER_ANY, hip.ORDER_BEST):
        idx = [torch.zeros((b * hkv, budget), dtype=torch.int32, device=DEV) for _ in range(2)]
        out = [torch.empty((b, hq, hd), dtype=torch.bfloat16, device=DEV) for _ in range(2)]
        hip.decode_layer(qd, kd, vd, p_len, hi, s_len, budget, None, idx[0], out[0], ws, order=order)
        call = hip.LayerCall(qd, kd, vd, p_len, hi, s_len, budget, None, idx[1], out[1], ws, order=order)
        assert call.route() == (hip.ROUTE_ONE_KERNEL if order == hip.ORDER_ANY else hip.ROUTE_STREAM)
        call(select_state_ready=True)
        call(select_state_ready=True)
        torch.cuda.synchronize()
        assert torch.equal(torch.sort(idx[0], dim=1).values, torch.sort(idx[1], dim=1).values)
        # (the one-kernel route deals rows to blocks in arrival order: equal within float rounding)
        assert torch.allclose(out[0].float(), out[1].float(), atol=2e-3, rtol=2.0 ** -7)


def test_a_sketch_moves_the_crossover_to_the_chain():
    """With a sketch the kernel chain is the faster one from about 40 Ki rows per unit on, so the
    one-kernel route ends there; without a sketch it goes on to 640 Ki rows in all.  Both routes
    select the same ids."""
    torch.manual_seed(306)
    b, hq, hkv, hd, budget = 1, 8, 2, 128, 512
    for n_ctx, want_with_sketch in ((40 * 1024 + 68, hip.ROUTE_ONE_KERNEL), (40 * 1024 + 69, hip.ROUTE_SKETCH)):
        kd = torch.randn((b, hkv, n_ctx, hd), device=DEV).to(torch.bfloat16)
        vd = torch.randn((b, hkv, n_ctx, hd), device=DEV).to(torch.bfloat16)
        qd = torch.randn((b, hq, hd), device=DEV).to(torch.bfloat16)
        lo, hi, s_len = 4, n_ctx - 64, 64
        sk = hip.Sketch(kd).build(kd, lo, hi - lo)
        ws = hip.alloc_workspace(hip.layer_workspace_bytes(b * hkv, hi - lo, budget, hq // hkv, hd, budget + 69), DEV)
        got = {}
        for name, sketch in (("plain", None), ("sketch", sk)):
            idx = torch.zeros((b * hkv, budget), dtype=torch.int32, device=DEV)
            out = torch.empty((b, hq, hd), dtype=torch.bfloat16, device=DEV)
            call = hip.LayerCall(qd, kd, vd, lo, hi, s_len, budget, None, idx, out, ws, sketch=sketch)
            assert call.route() == (hip.ROUTE_ONE_KERNEL if sketch is None else want_with_sketch), (n_ctx, name)
            call(select_state_ready=False)
            torch.cuda.synchronize()
            assert hip.last_route() == call.route()
            got[name] = (torch.sort(idx, dim=1).values.cpu(), out.float().cpu())
        assert torch.equal(got["plain"][0], got["sketch"][0]), n_ctx
        assert torch.allclose(got["plain"][1], got["sketch"][1], atol=2e-3, rtol=2.0 ** -7), n_ctx


@pytest.mark.parametrize("hd", [96, 80, 192])
def test_other_head_dims_run_zero_padded(hd):
    """Head dims between the supported ones: rows, queries and values zero-padded to the next
    supported size (a row stride of that size) and the softmax scale of the TRUE head dim give
    the ids and the attention of the unpadded problem on every route; the padded output columns
    come back zero."""
    rng = np.random.default_rng(400 + hd)
    pad = 128 if hd <= 128 else 256
    b, hq, hkv, budget, mode = 1, 8, 2, 300, 0
    g = hq // hkv
    for n_ctx, with_sketch, order, want_route in ((5000, False, hip.ORDER_ANY, hip.ROUTE_ONE_KERNEL),
                                                  (45000, True, hip.ORDER_ANY, hip.ROUTE_SKETCH),
                                                  (45000, False, hip.ORDER_BEST, hip.ROUTE_STREAM)):
        k, v, q = rand_bf16(rng, b, hkv, n_ctx, hd), rand_bf16(rng, b, hkv, n_ctx, hd), rand_bf16(rng, b, hq, hd)
        nk, nv = rand_bf16(rng, b, hkv, hd), rand_bf16(rng, b, hkv, hd)

        def padded(a):
            out = np.zeros(a.shape[:-1] + (pad,), dtype=np.uint16)
            out[..., :hd] = a
            return to_dev_bf16(out)

        kd, vd, qd, nkd, nvd = padded(k), padded(v), padded(q), padded(nk), padded(nv)
        p_len, s_len, lo, hi = orc.region_split(n_ctx, 4, 64)
        region = hi - lo
        sk = hip.Sketch(kd).build(kd, lo, region) if with_sketch else None
        ws = hip.alloc_workspace(hip.layer_workspace_bytes(b * hkv, region, budget, g, pad, budget + 69), DEV)
        idx = torch.full((b * hkv, budget), -1, dtype=torch.int32, device=DEV)
        out = torch.full((b, hq, pad), float("nan"), dtype=torch.bfloat16, device=DEV)
        hip.decode_layer(qd, kd, vd, p_len, hi, s_len, budget, None, idx, out, ws, nkd, nvd, mode=mode,
                         order=order, scale=1.0 / float(np.sqrt(hd)), sketch=sk)
        torch.cuda.synchronize()
        assert hip.last_route() == want_route, (hd, n_ctx)
        dense = hip.score(kd, qd, lo, region, mode, q_group=g).cpu().numpy()
        ids = idx.cpu().numpy().astype(np.int64)
        got = orc.bf16_to_f32(to_np_u16(out))
        assert not np.any(got[..., hd:]), hd
        for u in range(b * hkv):
            want = orc.topk_select(dense[u], budget, mode).astype(np.int64)
            assert np.array_equal(np.sort(ids[u]), np.sort(want)), (hd, n_ctx, u)
            # the scores of the padded rows are those of the unpadded ones (zeros add nothing)
            exact = orc.bf16_to_f32(k[0, u, lo:hi]).astype(np.float64) @ \
                orc.bf16_to_f32(orc.group_mean_bf16(q, hkv)[0, u]).astype(np.float64)
            assert np.all(np.abs(dense[u] - exact) <= 1e-5 * np.maximum(1.0, np.abs(exact)) + 1e-4), (hd, u)
            rows = np.concatenate([want + lo, np.arange(p_len), np.arange(hi, hi + s_len)]).astype(np.int64)
            o, _ = orc.sparse_attention(q[0, u * g:(u + 1) * g], k[0, u][rows], v[0, u][rows], nk[0, u], nv[0, u])
            assert bf16_close(got[0, u * g:(u + 1) * g, :hd], o), (hd, n_ctx, u)


def test_small_context_agrees_with_the_kernel_chain_on_random_cases():
    """120 random shapes, budgets, key modes and data laws: the one-kernel route (ids in any
    order) against the chain of kernels that the same call takes when the ids are asked best
    first.  Same id sets, outputs within bf16 rounding of each other."""
    rng = np.random.default_rng(306)
    n_one = 0
    for case in range(120):
        hd = int(rng.choice([64, 128, 256]))
        g = int(rng.choice([1, 2, 4, 7, 8]))
        hkv = int(rng.integers(1, 7))
        b = int(rng.integers(1, 4))
        p, s = int(rng.integers(0, 6)), int(rng.integers(0, 40))
        region = int(rng.choice([1, 2, 17, 255, 256, 257, 1000, 3000, 7000, 12000]))
        budget = int(rng.choice([1, 8, 100, 512, 2048, region, region + 5]))
        mode = int(rng.integers(0, 2))
        law = rng.choice(["normal", "integers", "constant", "two_values"])
        n_ctx = p + region + s
        shape = (b, hkv, n_ctx, hd)
        if law == "normal":
            kf = rng.standard_normal(shape)
        elif law == "integers":
            kf = rng.integers(-2, 3, shape)
        elif law == "constant":
            kf = np.broadcast_to(rng.standard_normal((b, hkv, 1, hd)), shape)
        else:
            kf = np.where(rng.random((b, hkv, n_ctx, 1)) < 0.5, 1.0, -1.0) * rng.standard_normal((b, hkv, 1, hd))
        k = to_dev_bf16(orc.f32_to_bf16(np.ascontiguousarray(kf, dtype=np.float32)))
        v = to_dev_bf16(rand_bf16(rng, *shape))
        q = to_dev_bf16(rand_bf16(rng, b, hkv * g, hd))
        nk, nv = to_dev_bf16(rand_bf16(rng, b, hkv, hd)), to_dev_bf16(rand_bf16(rng, b, hkv, hd))
        k_eff = min(budget, region)
        ws = hip.alloc_workspace(hip.layer_workspace_bytes(b * hkv, region, budget, g, hd, k_eff + p + s + 1), DEV)
        res = {}
        for order in (hip.ORDER_ANY, hip.ORDER_BEST):
            idx = torch.full((b * hkv, max(budget, 1)), -1, dtype=torch.int32, device=DEV)
            out = torch.empty((b, hkv * g, hd), dtype=torch.bfloat16, device=DEV)
            lse = torch.empty((b, hkv * g), dtype=torch.float32, device=DEV)
            args = (q, k, v, p, p + region, s, budget, None, idx, out, ws, nk, nv)
            kw = dict(lse=lse, mode=mode, order=order)
            route = hip.decode_layer_route(*args, **kw)
            hip.decode_layer(*args, **kw)
            hip.decode_layer_status(*args, **kw)
            res[order] = (torch.sort(idx[:, :k_eff], dim=1).values.cpu(), out.float().cpu(), lse.cpu(), route)
        one, chain = res[hip.ORDER_ANY], res[hip.ORDER_BEST]
        n_one += one[3] == hip.ROUTE_ONE_KERNEL
        tag = (case, hd, g, hkv, b, p, s, region, budget, mode, str(law))
        assert chain[3] != hip.ROUTE_ONE_KERNEL, tag
        assert torch.equal(one[0], chain[0]), tag
        assert torch.allclose(one[1], chain[1], atol=4e-3, rtol=2.0 ** -6), tag
        assert torch.allclose(one[2], chain[2], atol=1e-3, rtol=1e-4), tag
    assert n_one >= 100       # (a group size whose kernel does not fit twice on a CU takes the chain)
