"""Robustness of the fire kernels beyond the benchmark shapes: tensors whose element index does not
fit 32 bits (the reference indexes with ``int``: snnlib/cuda/snn_kernel_fp.cu:45, :60-63), capture into
a HIP graph with replays, and concurrent launches on two streams."""
import numpy as np
import pytest
import torch

from conftest import ALPHA, BETA, INTERVAL, THRESH

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cabi():
    from snn_gpu_training_bptt_amd import lif_cabi
    lif_cabi.load()
    return lif_cabi


def test_element_index_beyond_32_bits(cabi):
    """T=3 rows of 2**31 + 4096 neurons: the last row starts past element 2**32."""
    from oracle import c_oracle
    T, N = 3, (1 << 31) + 4096
    need = 4 * T * N * 4
    free, _ = torch.cuda.mem_get_info()
    if free < need + (8 << 30):
        pytest.skip(f"needs {need >> 30} GiB of device memory")
    gen = torch.Generator(device="cuda").manual_seed(77)
    x = torch.empty((T, 1, N), device="cuda")
    g = torch.empty((T, 1, N), device="cuda")
    for t in range(T):          # row-wise: keeps the generator's temporaries small
        x[t].normal_(0.5, 1.0, generator=gen)
        g[t].normal_(0.0, 1.0, generator=gen)
    spike = torch.empty_like(x)
    gx = torch.empty_like(x)
    cabi.fire_s_fp_into(x, spike, ALPHA, THRESH)
    cabi.fire_bp_into(x, g, gx, ALPHA, THRESH, BETA, INTERVAL)
    torch.cuda.synchronize()
    # neurons at both ends, around the 2**31 boundary and a random sample
    idx = torch.cat([torch.arange(0, 2048), torch.arange((1 << 31) - 1024, (1 << 31) + 1024),
                     torch.arange(N - 2048, N),
                     torch.randint(0, N, (50_000,), generator=torch.Generator().manual_seed(3))]).cuda()
    take = lambda t: t.view(T, N)[:, idx].cpu().numpy().reshape(T, 1, -1)
    _, spike_o = c_oracle.fire_forward(take(x), ALPHA, THRESH)
    gx_o = c_oracle.fire_backward(take(x), take(g), ALPHA, THRESH, BETA, INTERVAL)
    assert np.array_equal(take(spike), spike_o)
    assert np.array_equal(take(gx), gx_o)
    del x, g, spike, gx
    torch.cuda.empty_cache()


def test_hip_graph_capture_and_replay(cabi):
    """Forward + backward captured once, replayed with fresh inputs and eager work in between: every
    replay must equal the eager result (the entry points allocate nothing and record no memsets)."""
    from oracle import c_oracle
    shape = (8, 4, 64, 16, 16)
    gen = torch.Generator().manual_seed(78)
    x = torch.empty(shape, device="cuda")
    g = torch.empty(shape, device="cuda")
    spike = torch.empty_like(x)
    gx = torch.empty_like(x)
    x.copy_(0.5 + torch.randn(shape, generator=gen))
    g.copy_(torch.randn(shape, generator=gen))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):          # warm-up on the capture stream, as torch recommends
        cabi.fire_s_fp_into(x, spike, ALPHA, THRESH)
        cabi.fire_bp_into(x, g, gx, ALPHA, THRESH, BETA, INTERVAL)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cabi.fire_s_fp_into(x, spike, ALPHA, THRESH)
        cabi.fire_bp_into(x, g, gx, ALPHA, THRESH, BETA, INTERVAL)

    for rep in range(4):
        x_cpu = 0.5 + torch.randn(shape, generator=gen)
        g_cpu = torch.randn(shape, generator=gen)
        x.copy_(x_cpu)
        g.copy_(g_cpu)
        spike.fill_(-1.0)
        gx.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        _, spike_o = c_oracle.fire_forward(x_cpu.numpy(), ALPHA, THRESH)
        gx_o = c_oracle.fire_backward(x_cpu.numpy(), g_cpu.numpy(), ALPHA, THRESH, BETA, INTERVAL)
        assert np.array_equal(spike.cpu().numpy(), spike_o), f"replay {rep}: spikes"
        assert np.array_equal(gx.cpu().numpy(), gx_o), f"replay {rep}: gradients"
        # eager work between replays
        eager = torch.empty_like(x)
        cabi.fire_s_fp_into(x, eager, ALPHA, THRESH)
        assert torch.equal(eager, spike)


def test_two_streams_concurrently(cabi):
    from oracle import c_oracle
    shape = (8, 8, 64, 32, 32)
    gen = torch.Generator().manual_seed(79)
    data = []
    for _ in range(2):
        x_cpu = 0.5 + torch.randn(shape, generator=gen)
        g_cpu = torch.randn(shape, generator=gen)
        data.append((x_cpu, g_cpu, x_cpu.cuda(), g_cpu.cuda()))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = []
    for (x_cpu, g_cpu, x, g), st in zip(data, streams):
        with torch.cuda.stream(st):
            spike, gx = torch.empty_like(x), torch.empty_like(x)
            for _ in range(3):          # several rounds so the two streams overlap
                cabi.fire_s_fp_into(x, spike, ALPHA, THRESH)
                cabi.fire_bp_into(x, g, gx, ALPHA, THRESH, BETA, INTERVAL)
            outs.append((spike, gx))
    for st in streams:
        st.synchronize()
    for (x_cpu, g_cpu, _, _), (spike, gx) in zip(data, outs):
        _, spike_o = c_oracle.fire_forward(x_cpu.numpy(), ALPHA, THRESH)
        gx_o = c_oracle.fire_backward(x_cpu.numpy(), g_cpu.numpy(), ALPHA, THRESH, BETA, INTERVAL)
        assert np.array_equal(spike.cpu().numpy(), spike_o)
        assert np.array_equal(gx.cpu().numpy(), gx_o)


def test_events_attached_to_the_next_kernel(cabi):
    """snnlif_time_next_kernel: the armed events bracket exactly one launch, results are unchanged,
    the arming is consumed, and the duration is no longer than the interval between two stream
    markers around the same launch."""
    from oracle import c_oracle
    shape = (8, 16, 64, 32, 32)
    gen = torch.Generator().manual_seed(83)
    x_cpu = 0.5 + torch.randn(shape, generator=gen)
    g_cpu = torch.randn(shape, generator=gen)
    x, g = x_cpu.cuda(), g_cpu.cuda()
    spike, gx = torch.empty_like(x), torch.empty_like(x)
    for _ in range(3):
        cabi.fire_bp_into(x, g, gx, ALPHA, THRESH, BETA, INTERVAL)
    k0, k1, m0, m1, late = (torch.cuda.Event(enable_timing=True) for _ in range(5))
    for e in (k0, k1, late):
        e.record()
    torch.cuda.synchronize()
    gx.zero_()
    m0.record()
    cabi.time_next_kernel(k0, k1)
    cabi.fire_bp_into(x, g, gx, ALPHA, THRESH, BETA, INTERVAL)
    m1.record()
    # not armed any more: this launch must leave k0 / k1 alone
    cabi.fire_s_fp_into(x, spike, ALPHA, THRESH)
    late.record()
    torch.cuda.synchronize()
    kernel_ms, marker_ms = k0.elapsed_time(k1), m0.elapsed_time(m1)
    assert 0.0 < kernel_ms <= marker_ms * 1.02, (kernel_ms, marker_ms)
    assert k1.elapsed_time(late) > 0.0
    gx_o = c_oracle.fire_backward(x_cpu.numpy(), g_cpu.numpy(), ALPHA, THRESH, BETA, INTERVAL)
    _, spike_o = c_oracle.fire_forward(x_cpu.numpy(), ALPHA, THRESH)
    assert np.array_equal(gx.cpu().numpy(), gx_o)
    assert np.array_equal(spike.cpu().numpy(), spike_o)
    # disarming with two NULLs is accepted
    cabi.time_next_kernel(None, None)
    cabi.fire_s_fp_into(x, spike, ALPHA, THRESH)
    torch.cuda.synchronize()
    assert np.array_equal(spike.cpu().numpy(), spike_o)


def test_stop_events_alone_give_completion_intervals_that_add_up(cabi):
    """How bench.py times its kernels: a stop event on every dispatch and no start event.  The interval
    between two consecutive completions is positive, the intervals of a sequence of launches add up to the
    interval between the first and the last completion, and that is no longer than the span between two
    stream markers around the sequence."""
    x = (0.5 + torch.randn(8, 16, 64, 32, 32)).cuda()
    g = torch.randn_like(x)
    spike, gx = torch.empty_like(x), torch.empty_like(x)
    n = 6
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(2 * n)]
    m0, m1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for e in stops:
        e.record()
    cabi.fire_s_fp_into(x, spike, ALPHA, THRESH)   # warm-up
    torch.cuda.synchronize()
    m0.record()
    for i in range(n):
        cabi.time_next_kernel(None, stops[2 * i])
        cabi.fire_s_fp_into(x, spike, ALPHA, THRESH)
        cabi.time_next_kernel(None, stops[2 * i + 1])
        cabi.fire_bp_into(x, g, gx, ALPHA, THRESH, BETA, INTERVAL)
    m1.record()
    torch.cuda.synchronize()
    spans = [stops[i - 1].elapsed_time(stops[i]) for i in range(1, 2 * n)]
    assert all(ms > 0.0 for ms in spans), spans
    total = stops[0].elapsed_time(stops[-1])
    assert abs(sum(spans) - total) <= 1e-3 * total + 2e-3, (sum(spans), total)
    assert total <= m0.elapsed_time(m1) * 1.02


def test_an_armed_timer_does_not_outlive_a_failed_call(cabi):
    """An entry point that returns an argument error consumes the arming: the events must not end up
    on the next, unrelated launch."""
    lib = cabi.load()
    x = (0.5 + torch.randn(8, 8, 64, 32, 32)).cuda()
    spike = torch.empty_like(x)
    k0, k1, after = (torch.cuda.Event(enable_timing=True) for _ in range(3))
    k0.record()
    k1.record()
    torch.cuda.synchronize()
    cabi.time_next_kernel(k0, k1)
    assert lib.snnlif_fire_s_fp(x.data_ptr(), spike.data_ptr(), 9, 8, x.numel() // 8, ALPHA, THRESH, None) == cabi.ERR_DTYPE
    for _ in range(3):                                   # were the timer still armed, k1 would now be
        cabi.fire_s_fp_into(x, spike, ALPHA, THRESH)     # re-recorded at the end of the first of these
    after.record()
    torch.cuda.synchronize()
    first_kernel_end_to_after = k1.elapsed_time(after)
    singles = []
    for _ in range(3):      # one launch, best of three: a hiccup in one run must not decide the test
        cabi.time_next_kernel(k0, k1)
        cabi.fire_s_fp_into(x, spike, ALPHA, THRESH)
        torch.cuda.synchronize()
        singles.append(k0.elapsed_time(k1))
    one_kernel = min(singles)
    # k1 kept its original record (before all three launches): all three lie between it and `after`
    assert first_kernel_end_to_after > 2.0 * one_kernel, (first_kernel_end_to_after, singles)


def test_events_bracket_the_whole_of_a_multi_kernel_operation(cabi):
    """The batch-norm backward is three kernels: the armed events are recorded before the first and
    after the last, so they cover at least the two sweeps."""
    shape = (8, 16, 32, 32, 32)
    T, B, C, HW = 8, 16, 32, 1024
    x = (0.5 + torch.randn(shape)).cuda()
    g = torch.randn(shape).cuda()
    w, b = torch.ones(C, device="cuda"), torch.zeros(C, device="cuda")
    var, mean = torch.ones(C, device="cuda"), torch.full((C,), 0.5, device="cuda")
    ivar, spike = torch.empty_like(var), torch.empty_like(x)
    cabi.bn_fire_s_fp_into(x, w, b, var, mean, ivar, spike, 1e-5, ALPHA, THRESH)
    gx, gw, gb = torch.empty_like(x), torch.empty_like(w), torch.empty_like(w)
    ws = torch.empty(cabi.bn_fire_bp_workspace_bytes(cabi.DTYPE_F32, T, B, C, HW), dtype=torch.uint8, device="cuda")
    e = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
    for ev in e:
        ev.record()
    torch.cuda.synchronize()
    for _ in range(2):
        cabi.bn_fire_bp_into(x, w, b, ivar, mean, g, gx, gw, gb, ALPHA, THRESH, BETA, INTERVAL, ws)
    cabi.time_next_kernel(e[0], e[1])
    cabi.bn_fire_bp_into(x, w, b, ivar, mean, g, gx, gw, gb, ALPHA, THRESH, BETA, INTERVAL, ws)
    torch.cuda.synchronize()
    whole = e[0].elapsed_time(e[1])
    sweeps = []
    for _ in range(3):      # the second sweep alone, best of three: a hiccup in one run must not decide the test
        cabi.time_next_kernel(e[2], e[3])
        cabi.bn_fire_bp_dist2_into(x, w, b, ivar, mean, g, gw, gb, gx, ALPHA, THRESH, BETA, INTERVAL)
        torch.cuda.synchronize()
        sweeps.append(e[2].elapsed_time(e[3]))
    one_sweep = min(sweeps)
    # sweep 1 moves 8 bytes per neuron-step and sweep 2 twelve: the whole is about 1.7 sweeps 2
    assert whole > 1.3 * one_sweep, (whole, sweeps)


def test_layers_captured_with_torch_cuda_graph():
    """A forward + backward through the PyTorch-facing layers (Fire, then BnFire with given statistics,
    whose backward draws its workspace from the caching allocator) captured by torch.cuda.graph and
    replayed with fresh inputs; every replay equals the eager result of the same layers."""
    from snn_gpu_training_bptt_amd import snnlib_func as sf
    saved = (sf.alpha, sf.thresh, sf.beta, sf.interval)
    sf.alpha, sf.thresh, sf.beta, sf.interval = ALPHA, THRESH, BETA, INTERVAL
    try:
        shape = (6, 4, 16, 8, 8)
        C = shape[2]
        gen = torch.Generator().manual_seed(84)
        w = (0.5 + torch.rand(C, generator=gen)).cuda().requires_grad_(True)
        b = (0.2 * torch.randn(C, generator=gen)).cuda().requires_grad_(True)
        var = (0.5 + torch.rand(C, generator=gen)).cuda()
        mean = (0.1 * torch.randn(C, generator=gen)).cuda()
        x = torch.zeros(shape, device="cuda", requires_grad=True)
        gout = torch.zeros(shape, device="cuda")

        def run():
            spikes = sf.fire_func(x)
            out = sf.bn_fire_func(spikes * 1.5 - 0.2, w, b, var, mean, (0, 1, 3, 4), 1e-5)
            gx, gw, gb = torch.autograd.grad(out, (x, w, b), gout)
            return out, gx, gw, gb

        def load(seed):
            g2 = torch.Generator().manual_seed(seed)
            with torch.no_grad():
                x.copy_(0.5 + torch.randn(shape, generator=g2))
                gout.copy_(torch.randn(shape, generator=g2))

        load(0)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                run()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()

        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static = run()
        for seed in (1, 2, 3, 4):
            load(seed)
            graph.replay()
            torch.cuda.synchronize()
            got = [t.clone() for t in static]
            want = run()                      # eager work between the replays
            torch.cuda.synchronize()
            for name, a, e in zip(("out", "grad x", "grad weight", "grad bias"), got, want):
                assert torch.equal(a, e), f"replay with seed {seed}: {name}"
    finally:
        sf.alpha, sf.thresh, sf.beta, sf.interval = saved


def test_host_threads_launching_concurrently(cabi):
    """Four host threads, each with its own stream and tensors, calling the C ABI at the same time
    (ctypes drops the GIL for the duration of a call): the library keeps no shared state, and the
    timing hook of one thread must not leak into another's launches."""
    import threading
    from oracle import c_oracle
    shape = (6, 4, 32, 16, 16)
    results, errors = {}, []
    start = threading.Barrier(4)

    def worker(idx):
        try:
            gen = torch.Generator().manual_seed(90 + idx)
            x_cpu = 0.5 + torch.randn(shape, generator=gen)
            g_cpu = torch.randn(shape, generator=gen)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                x, g = x_cpu.cuda(), g_cpu.cuda()
                spike, gx = torch.empty_like(x), torch.empty_like(x)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                e1.record()
                start.wait()
                for it in range(20):
                    if idx == 0 and it == 10:        # only this thread arms the hook
                        cabi.time_next_kernel(e0, e1)
                    cabi.fire_s_fp_into(x, spike, ALPHA, THRESH)
                    cabi.fire_bp_into(x, g, gx, ALPHA, THRESH, BETA, INTERVAL)
                stream.synchronize()
            results[idx] = (x_cpu, g_cpu, spike.cpu(), gx.cpu(), e0.elapsed_time(e1) if idx == 0 else None)
        except Exception as exc:  # surfaced in the main thread below
            errors.append((idx, repr(exc)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
    assert not errors, errors
    assert sorted(results) == [0, 1, 2, 3]
    for idx, (x_cpu, g_cpu, spike, gx, ms) in results.items():
        _, spike_o = c_oracle.fire_forward(x_cpu.numpy(), ALPHA, THRESH)
        gx_o = c_oracle.fire_backward(x_cpu.numpy(), g_cpu.numpy(), ALPHA, THRESH, BETA, INTERVAL)
        assert np.array_equal(spike.numpy(), spike_o), f"thread {idx}: spikes"
        assert np.array_equal(gx.numpy(), gx_o), f"thread {idx}: gradients"
    assert results[0][4] > 0.0
