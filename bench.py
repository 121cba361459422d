"""Headline benchmark: one SO3Convolution layer, forward + backward, fp32, b_in = b_out = 32,
64 -> 64 features, batch 16, default near-identity grid (192 points), Kaiming-normal kernel,
loss = sum(out^2) - benchmark config "Single SO3Convolution layer".  One step = one forward +
backward over one synthetic batch that is already resident in HBM.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-fft]

Prints ONE JSON line.  `roofline` is for the dominant kernel (the block-diagonal spectral
product so3_mm, bound by the fp32 matrix cores), timed with events on the launch stream inside
the timed steps; `so3_fft` reports the standalone SO(3) FFT round trip of benchmark config 2
against HBM bandwidth; `cpu_baseline` is the CPU oracle timed on this host on a bounded sample.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3   # MI355X dense fp32 matrix
PEAK_HBM_GBS = 8000.0           # MI355X HBM3E
# HBM-side bytes per launch of the three product kernels at this workload, from rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE scaled by a 1 GiB elementwise kernel of the same run (profiles/so3_mm_real_b32_B16_F64_hbm_traffic.md);
# not re-measured at run time.
MM_TRAFFIC_BYTES = {"s2cnn_so3_mm_real_fwd": 6.67e9 + 0.179e9, "s2cnn_so3_mm_real_gradx": 6.61e9 + 0.179e9,
                    "s2cnn_so3_mm_real_grady": 5.04e9 + 0.716e9}


def sum_of_squares(t):
    """The loss of benchmark config 4, sum(out^2), with its gradient 2 out written out by hand: one reduction pass
    forward and one elementwise pass backward over the 1 GiB output.  (Autograd through out * out or
    vector_norm(out)**2 is the same function with three to five passes, none of them the layer's.)"""
    import torch
    from s2cnn_amd import _hip

    def timed(name, fn):
        """fn() between two events on the launch stream while a KernelTimer is active: the loss is the harness's own
        work, and its time is reported under its own keys beside the library's calls."""
        timer = _hip.KernelTimer.active
        if timer is None or not torch.cuda.is_available():
            return fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        out = fn()
        e1.record()
        timer.records.append((name, e0, e1))
        return out

    class _SumOfSquares(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x):
            ctx.save_for_backward(x)
            return timed("harness_loss_forward", lambda: torch.linalg.vector_norm(x).square())

        @staticmethod
        def backward(ctx, g):
            (x,) = ctx.saved_tensors
            return timed("harness_loss_backward", lambda: x * (2.0 * g))

    return _SumOfSquares.apply(t)


def nspec(b):
    return b * (4 * b * b - 1) // 3


def mm_flops(nl, B, Fi, Fo, real=True):
    """Algorithmic flops of one block product: B Fi Fo sum_l (2l+1)^3 = B Fi Fo nl^2 (2 nl^2 - 1) multiply-adds,
    real (2 flops each) in the real basis the layer uses, complex (8 flops each) in so3_mm proper.  The complex kernels
    form a complex product from three real ones, so the matrix cores execute 6 flops per complex multiply-add: their
    `frac` is that executed fraction, and `algorithmic_frac` (4/3 of it) the textbook count."""
    return (2.0 if real else 8.0) * B * Fi * Fo * nl * nl * (2 * nl * nl - 1)


def so3_fft_bytes(b_in, b_out, n):
    """Algorithmic bytes of one SO(3) transform: real grid + complex spectrum."""
    return 4.0 * n * (2 * b_in) ** 3 + 8.0 * n * nspec(b_out)


def measure_rows(torch, dev, with_cpu):
    """Every other op of the path at its benchmark-config size: GPU time (events on the launch stream), the
    algorithmic bytes or flops, the roofline fraction, and the CPU oracle on a bounded sample beside it."""
    import s2cnn_amd
    from s2cnn_amd import _hip
    from s2cnn_amd.soft import s2_fft as PS2
    from s2cnn_amd.soft import so3_fft as PSO3
    from oracle import cpu_path as O

    def gpu_ms(fn, reps=5):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    def cpu_s(fn):
        if not with_cpu:
            return None
        t0 = time.perf_counter()
        fn()
        return time.perf_counter() - t0

    rows = {}

    def add(name, ms, work, unit, cpu_t, cpu_frac, note):
        rate = work / (ms * 1e-3)
        if unit == "B":
            ent = {"ms": round(ms, 4), "bound": "hbm", "achieved_GBs": round(rate / 1e9, 1), "frac": round(rate / 1e9 / PEAK_HBM_GBS, 4)}
        else:
            ent = {"ms": round(ms, 4), "bound": "mfma", "achieved_TFLOPs": round(rate / 1e12, 2),
                   "frac": round(rate / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4)}
        if cpu_t is not None:
            ent["cpu_s_full_size_estimate"] = round(cpu_t / cpu_frac, 3)
            ent["cpu_sample"] = note
        rows[name] = ent

    g = torch.Generator().manual_seed(11)
    # --- S^2 ops at config-5 sizes: x [32, 6, 256, 256] -> [1024, 192, 2]; s2_mm 6 -> 100 features at nl = 32
    B5, Fi5, Fo5, b5i, b5o = 32, 6, 100, 128, 32
    xs2 = torch.rand(B5, Fi5, 2 * b5i, 2 * b5i, generator=g)
    xs2g = xs2.to(dev)
    s2spec = PS2.s2_rfft(xs2g, b_out=b5o)
    by = 4.0 * xs2.numel() + 8.0 * s2spec.numel() / 2
    t = cpu_s(lambda: O.s2_fft(O.as_complex(xs2[:4]), b_out=b5o))
    add("s2_analysis [32,6,256,256]->b32", gpu_ms(lambda: PS2.s2_rfft(xs2g, b_out=b5o)), by, "B", t, 4 / B5, "batch 4 of 32")
    gspec = torch.randn_like(s2spec)
    t = cpu_s(lambda: O.s2_ifft(gspec[:, :4].cpu(), for_grad=True, b_out=b5i))
    add("s2_synthesis b32->[32,6,256,256]", gpu_ms(lambda: PS2.s2_rifft(gspec, for_grad=True, b_out=b5i)), by, "B", t, 4 / B5, "batch 4 of 32")
    xk = torch.randn(b5o * b5o, B5, Fi5, 2, generator=g)
    yk = torch.randn(b5o * b5o, Fi5, Fo5, 2, generator=g)
    xkg, ykg = xk.to(dev).requires_grad_(), yk.to(dev).requires_grad_()
    zk = s2cnn_amd.s2_mm(xkg, ykg)
    gzk = torch.randn_like(zk)
    zbytes = 4.0 * zk.numel()
    t = cpu_s(lambda: O.s2_mm(xk[:, :2], yk))
    add("s2_mm fwd nl=32 B=32 6->100", gpu_ms(lambda: s2cnn_amd.s2_mm(xkg, ykg)), zbytes + 4.0 * (xk.numel() + yk.numel()), "B", t, 2 / B5, "batch 2 of 32")
    add("s2_mm grad (x and y)", gpu_ms(lambda: torch.autograd.grad(zk, (xkg, ykg), gzk, retain_graph=True)),
        2 * zbytes + 4.0 * 2 * (xk.numel() + yk.numel()), "B", None, 1, "")
    # the same product on real-basis spectra (what S2Convolution runs): half the bytes
    xr, yr = torch.randn(b5o * b5o, B5, Fi5, device=dev).requires_grad_(), torch.randn(b5o * b5o, Fi5, Fo5, device=dev).requires_grad_()
    zr = s2cnn_amd.s2_mm_real(xr, yr)
    gzr = torch.randn_like(zr)
    add("s2_mm_real fwd nl=32 B=32 6->100", gpu_ms(lambda: s2cnn_amd.s2_mm_real(xr, yr)), 4.0 * (zr.numel() + xr.numel() + yr.numel()), "B", None, 1, "")
    add("s2_mm_real grad (x and y)", gpu_ms(lambda: torch.autograd.grad(zr, (xr, yr), gzr, retain_graph=True)),
        4.0 * 2 * (zr.numel() + xr.numel() + yr.numel()), "B", None, 1, "")
    del zk, gzk, xkg, ykg, s2spec, gspec, xs2g, xr, yr, zr, gzr
    # --- the complex block product alone (config 3): x [43680, 16, 64, 2], y [43680, 64, 64, 2], forward and both gradients
    xm = (torch.randn(nspec(32), 16, 64, 2, generator=g) * 0.125)
    xmg = xm.to(dev).requires_grad_()
    ymg = (torch.randn(nspec(32), 64, 64, 2, device=dev) * 0.125).requires_grad_()
    zm = s2cnn_amd.so3_mm(xmg, ymg)
    gzm = torch.randn_like(zm)
    fl = mm_flops(32, 16, 64, 64, real=False)
    t = cpu_s(lambda: O.so3_mm(xm[:, :1], ymg.detach().cpu()))
    add("so3_mm fwd nl=32 B=16 64->64", gpu_ms(lambda: s2cnn_amd.so3_mm(xmg, ymg)), fl, "F", t, 1 / 16, "batch 1 of 16")
    add("so3_mm grad (x and y)", gpu_ms(lambda: torch.autograd.grad(zm, (xmg, ymg), gzm, retain_graph=True)), 2 * fl, "F", None, 1, "")
    for k in ("so3_mm fwd nl=32 B=16 64->64", "so3_mm grad (x and y)"):   # three real products per complex one: see measure_so3_mm
        rows[k]["algorithmic_frac"] = rows[k]["frac"]
        rows[k]["frac"] = round(0.75 * rows[k]["frac"], 4)
    del xm, xmg, ymg, zm, gzm
    # --- the real-basis product at the sizes of the second layer of config 5 (22 degrees, batch 32, 100 -> 100 features: blocks
    # of 100 do not divide the contraction stage of 32) and of the headline layer, one row per product
    from s2cnn_amd import so3_real
    for (nlr, Br, Fr) in ((22, 32, 100), (32, 16, 64)):
        xr = torch.randn(nspec(nlr), Br, Fr, device=dev).requires_grad_()
        yr = (torch.randn(nspec(nlr), Fr, Fr, device=dev) * 0.125).requires_grad_()
        gzr = torch.randn(nspec(nlr), Br, Fr, device=dev)

        def prod_step():
            zz = so3_real.so3_mm_real(xr, yr)
            torch.autograd.grad(zz, (xr, yr), gzr)

        for _ in range(2):
            prod_step()
        torch.cuda.synchronize()
        with _hip.KernelTimer() as kt:
            for _ in range(5):
                prod_step()
            torch.cuda.synchronize()
        flr = mm_flops(nlr, Br, Fr, Fr, real=True)
        for name, v in kt.summary().items():
            add("%s nl=%d B=%d %d->%d" % (name.replace("s2cnn_", ""), nlr, Br, Fr, Fr), sum(v) / len(v), flr, "F", None, 1, "")
        del xr, yr, gzr
    # --- Haar integral at config-4 output size [16, 64, 64, 64, 64]
    xi = torch.randn(16, 64, 64, 64, 64, device=dev)
    t = cpu_s(lambda: O.so3_integrate(xi[:2].cpu()))
    add("so3_integrate [16,64,64^3]", gpu_ms(lambda: s2cnn_amd.so3_integrate(xi)), 4.0 * xi.numel(), "B", t, 2 / 16, "batch 2 of 16")
    del xi
    # --- complex SO(3) transforms (so3_fft / so3_ifft) at b = 32, 16 volumes
    xc = torch.randn(16, 64, 64, 64, 2, device=dev)
    sc = PSO3.so3_fft(xc)
    byc = 4.0 * xc.numel() + 4.0 * sc.numel()
    t = cpu_s(lambda: O.so3_fft(xc[:1].cpu()))
    add("so3_fft complex b=32 N=16", gpu_ms(lambda: PSO3.so3_fft(xc)), byc, "B", t, 1 / 16, "1 volume of 16")
    t = cpu_s(lambda: O.so3_ifft(sc[:, :1].cpu()))
    add("so3_ifft complex b=32 N=16", gpu_ms(lambda: PSO3.so3_ifft(sc)), byc, "B", t, 1 / 16, "1 volume of 16")
    del xc, sc
    # --- real SO(3) transforms on the grids below 64^3, spectrum in the real basis as inside the layers: the 44^3 grid of
    # config 5 (b = 22, 32 x 100 volumes) and the 32^3 and 20^3 grids of the reference's SHREC17 model (b = 16 and 10,
    # 32 x 100 volumes)
    for bs, nv in ((22, 3200), (16, 3200), (10, 3200)):
        xs = torch.randn(nv, 2 * bs, 2 * bs, 2 * bs, device=dev)
        rs = PSO3.so3_rfft_real_basis(xs)
        bys = 4.0 * xs.numel() + 4.0 * rs.numel()
        t = cpu_s(lambda: O.so3_rfft(xs[:4].cpu()))
        add("so3 analysis real b=%d N=%d" % (bs, nv), gpu_ms(lambda: PSO3.so3_rfft_real_basis(xs)), bys, "B", t, 4 / nv, "4 volumes of %d" % nv)
        t = cpu_s(lambda: O.so3_rifft(O.so3_rfft(xs[:4].cpu())))
        add("so3 synthesis real b=%d N=%d" % (bs, nv), gpu_ms(lambda: PSO3.so3_rifft_real_basis(rs)), bys, "B", t, 4 / nv, "4 volumes of %d (with their analysis)" % nv)
        del xs, rs
    # --- kernel -> spectrum at config-4 size: [64, 64, 192] -> [43680, 64, 64, 2]
    grid = s2cnn_amd.so3_near_identity_grid()
    kk = torch.randn(64, 64, len(grid), device=dev)
    s2cnn_amd.so3_rft(kk, 32, grid)
    t = cpu_s(lambda: O.so3_rft(kk[:8].cpu(), 32, grid))
    # factorised over the 3 distinct betas of the grid: bound by writing the spectrum (8 B per complex entry), not by flops
    add("so3_rft [64,64,192]->b32", gpu_ms(lambda: s2cnn_amd.so3_rft(kk, 32, grid)), 8.0 * 64 * 64 * nspec(32) + 4.0 * kk.numel(), "B", t, 8 / 64,
        "8 of 64 input features")
    from s2cnn_amd.so3_real import so3_rft_real
    add("so3_rft_real (inside the layer)", gpu_ms(lambda: so3_rft_real(kk, 32, grid)), 4.0 * 64 * 64 * nspec(32) + 4.0 * kk.numel(), "B", None, 1, "")
    torch.cuda.empty_cache()
    return rows


def measure_so3_mm(torch, dev, reps=5):
    """Benchmark config 3: the complex block product alone, x [43680, 16, 64, 2], y [43680, 64, 64, 2] with entries
    N(0, 1/64), forward and the gradients with respect to x and y, each timed with events on the launch stream.  The kernels
    form a complex product from three real ones (6 flops per complex multiply-add on the matrix cores instead of 8), so
    `frac` = EXECUTED flops over the fp32 matrix peak (what the roofline bounds); `algorithmic_frac` counts the 8 flops of
    the textbook complex multiply-add and can exceed 1."""
    import s2cnn_amd
    from s2cnn_amd import _hip
    nl, B, Fi, Fo = 32, 16, 64, 64
    g = torch.Generator(device=dev).manual_seed(3)
    x = (torch.randn(nspec(nl), B, Fi, 2, device=dev, generator=g) * 0.125).requires_grad_()
    y = (torch.randn(nspec(nl), Fi, Fo, 2, device=dev, generator=g) * 0.125).requires_grad_()
    gz = torch.randn(nspec(nl), B, Fo, 2, device=dev, generator=g)

    def step():
        z = s2cnn_amd.so3_mm(x, y)
        torch.autograd.grad(z, (x, y), gz)

    for _ in range(2):
        step()
    torch.cuda.synchronize()
    with _hip.KernelTimer() as kt:
        for _ in range(reps):
            step()
        torch.cuda.synchronize()
    pc = {k: sum(v) / len(v) for k, v in kt.summary().items()}
    fl = mm_flops(nl, B, Fi, Fo, real=False)
    out = {"workload": "so3_mm fwd + grad x + grad y, x [43680,16,64,2], y [43680,64,64,2] (benchmark config 3)", "bound": "mfma",
           "flop_per_launch": fl, "executed_flop_per_launch": 0.75 * fl, "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s"}
    total = 0.0
    for name in ("s2cnn_so3_mm_fwd", "s2cnn_so3_mm_gradx", "s2cnn_so3_mm_grady"):
        ach = fl / (pc[name] * 1e-3) / 1e12
        total += pc[name]
        out[name] = {"ms": round(pc[name], 3), "achieved": round(0.75 * ach, 2), "frac": round(0.75 * ach / PEAK_FP32_MFMA_TFLOPS, 4),
                     "algorithmic_tflops": round(ach, 2), "algorithmic_frac": round(ach / PEAK_FP32_MFMA_TFLOPS, 4)}
    out["ms_fwd_bwd"] = round(total, 3)
    del x, y, gz
    torch.cuda.empty_cache()
    return out


def measure_network(torch, dev, steps, warmup, separate_relu=True):
    """The SHREC17-shaped network of benchmark config 5 (S2Conv 6->100 b 128->32, ReLU, SO3Conv 100->100 b 32->22, ReLU,
    SO3Conv 100->55 b 22->7, so3_integrate; batch 32, near-identity grids scaled by the bandwidth ratio), forward and
    backward with respect to the weights, timed like the headline step; time inside library calls listed beside it.
    Timed twice: with the activations inside the layers (activation="relu") and, as the reference's models are written,
    as separate torch.relu calls on the layers' outputs; both are the same function."""
    import math

    import s2cnn_amd
    from s2cnn_amd import _hip
    g1 = s2cnn_amd.s2_near_identity_grid(max_beta=math.pi / 8 * 30 / 128, n_alpha=8, n_beta=3)
    g2 = s2cnn_amd.so3_near_identity_grid(max_beta=math.pi / 8 * 30 / 32, max_gamma=2 * math.pi, n_alpha=8, n_beta=3, n_gamma=8)
    g3 = s2cnn_amd.so3_near_identity_grid(max_beta=math.pi / 8 * 30 / 22, max_gamma=2 * math.pi, n_alpha=8, n_beta=3, n_gamma=8)
    from s2cnn_amd.harness import smooth_spherical_batch
    x = smooth_spherical_batch(32, 6, 128, dev, seed=5)     # uniform-range values with smooth structure of degrees l < 16 plus noise

    def timed(activation):
        torch.manual_seed(8)
        c1 = s2cnn_amd.S2Convolution(6, 100, 128, 32, g1, activation=activation).to(dev)
        c2 = s2cnn_amd.SO3Convolution(100, 100, 32, 22, g2, activation=activation).to(dev)
        c3 = s2cnn_amd.SO3Convolution(100, 55, 22, 7, g3).to(dev)
        params = [q for c in (c1, c2, c3) for q in c.parameters()]
        act = torch.relu if activation is None else (lambda t: t)

        def step():
            for q in params:
                q.grad = None
            out = s2cnn_amd.so3_integrate(c3(act(c2(act(c1(x))))))
            sum_of_squares(out).backward()

        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / steps * 1e3
        with _hip.KernelTimer() as kt:
            step()
            torch.cuda.synchronize()
        calls = {k: round(sum(v), 3) for k, v in sorted(kt.summary().items(), key=lambda kv: -sum(kv[1]))}
        del c1, c2, c3, params
        torch.cuda.empty_cache()
        return ms, calls

    ms, calls = timed("relu")
    out = {"workload": "S2Conv 6->100 (b 128->32), SO3Conv 100->100 (32->22), SO3Conv 100->55 (22->7), integrate; batch 32, fwd+bwd (benchmark config 5)",
           "steps": steps, "ms_per_step": round(ms, 3), "samples_per_s": round(32 / (ms * 1e-3), 1),
           "library_ms": round(sum(v for k, v in calls.items() if k.startswith("s2cnn_")), 3), "library_calls_ms": calls}
    if separate_relu:
        ms_sep, calls_sep = timed(None)
        out["separate_relu"] = {"ms_per_step": round(ms_sep, 3),
                                "library_ms": round(sum(v for k, v in calls_sep.items() if k.startswith("s2cnn_")), 3)}
    return out


def measure_config1(torch, dev, reps=50):
    """Benchmark config 1: the digit network of examples/mnist/run.py:55-98 (S2Conv 1->20 b 30->10, ReLU, SO3Conv 20->40
    b 10->6, ReLU, so3_integrate, Linear 40->10), forward only, batch 32, input uniform in [0, 1) with 70 % zeros.  Timed
    eagerly (bound by its launches) and as one HIP graph replayed (nothing on the path allocates through HIP, synchronises or
    records a memset)."""
    from s2cnn_amd import _hip, harness
    torch.manual_seed(0)
    net = harness.S2ConvNet_original().to(dev).eval()
    g = torch.Generator().manual_seed(1)
    x = (torch.rand(32, 1, 60, 60, generator=g) * (torch.rand(32, 1, 60, 60, generator=g) < 0.3)).to(dev)

    def wall_ms(fn):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps * 1e3

    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                net(x)                                  # tables, workspaces and allocator pools exist before the capture
        torch.cuda.current_stream().wait_stream(side)
        eager = wall_ms(lambda: net(x))
        with _hip.KernelTimer() as kt:
            net(x)
            torch.cuda.synchronize()
        library = sum(sum(v) for k, v in kt.summary().items())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_y = net(x)
        replay = wall_ms(graph.replay)
        same = bool(torch.equal(static_y, net(x)))
    return {"workload": "S2Conv 1->20 (b 30->10), ReLU, SO3Conv 20->40 (b 10->6), ReLU, integrate, Linear 40->10; batch 32, forward "
                        "(benchmark config 1)",
            "eager_ms": round(eager, 4), "eager_samples_per_s": round(32 / (eager * 1e-3), 1), "library_ms": round(library, 4),
            "graph_replay_ms": round(replay, 4), "graph_replay_samples_per_s": round(32 / (replay * 1e-3), 1),
            "replay_equals_eager": same}


def measure_overlap(torch, dev, reps=6):
    """Can the transforms (bound by vector instructions and latency) and the products (bound by the matrix cores) of the
    headline layer share the chip?  Half of the layer's batch each: the analysis of 512 volumes of 64^3 and the real-basis
    product at batch 8 (64 -> 64 features, 32 degrees), first one after the other on one stream, then at the same time on two
    streams of equal priority.  A compute unit cannot hold a workgroup of both kernels at once (registers and LDS, see
    profiles/), so the two can only divide the CUs between them."""
    import s2cnn_amd
    from s2cnn_amd.soft import so3_fft as PSO3
    nl, B, F = 32, 8, 64
    x = torch.randn(B * F, 64, 64, 64, device=dev)
    xs = torch.randn(nspec(nl), B, F, device=dev)
    ys = torch.randn(nspec(nl), F, F, device=dev) * 0.125
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()

    def both(parallel):
        a, b = (s1, s2) if parallel else (s1, s1)
        with torch.cuda.stream(a):
            PSO3.so3_rfft_real_basis(x)
        with torch.cuda.stream(b):
            s2cnn_amd.so3_mm_real(xs, ys)

    def timed(fn):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps * 1e3

    def only_fft():
        with torch.cuda.stream(s1):
            PSO3.so3_rfft_real_basis(x)

    def only_mm():
        with torch.cuda.stream(s1):
            s2cnn_amd.so3_mm_real(xs, ys)

    out = {"workload": "analysis of 512 volumes of 64^3 and so3_mm_real forward at batch 8 (64->64, 32 degrees): half of the headline layer's batch each",
           "analysis_alone_ms": round(timed(only_fft), 4), "product_alone_ms": round(timed(only_mm), 4),
           "one_stream_ms": round(timed(lambda: both(False)), 4), "two_streams_ms": round(timed(lambda: both(True)), 4)}
    out["gain_of_two_streams"] = round(1.0 - out["two_streams_ms"] / out["one_stream_ms"], 4)
    return out


def measure_fft_floor(torch, dev, nvol=256, reps=10):
    """What the plane pipeline of the per-volume 64^3 kernels costs without the Wigner contraction: the shipped kernels
    with parts compiled out (s2cnn_so3_fft64_probe of the measurement library libs2cnn_probe.so, built by
    `python -m s2cnn_amd.csrc.build --probes`; the results of the stripped variants are meaningless), timed with
    events on the launch stream at the size of benchmark config 2.  The passes between records and spectral rows are
    timed from the full transforms (they are the difference between the transform and its kernel)."""
    from s2cnn_amd import _hip
    from s2cnn_amd.soft import so3_fft as PSO3
    b = 32
    x = torch.randn(nvol, 64, 64, 64, generator=torch.Generator().manual_seed(3)).to(dev)
    y = torch.empty_like(x)
    L = _hip.lib()
    P = _hip.probe_lib()
    ws = _hip.workspace(L.s2cnn_so3_analysis_workspace(b, b, nvol, 0), x.device)
    packed = {0: PSO3._setup_packed_wigner(b, b, True, False, x.device), 1: PSO3._setup_packed_wigner(b, b, False, True, x.device)}
    spec = PSO3.so3_rfft(x)
    out = {}
    variants = [("analysis kernel", 0, 0), ("analysis kernel, no contraction multiply-adds", 0, 1),
                ("analysis kernel, no contraction and no table loads", 0, 2),
                ("synthesis kernel", 1, 0), ("synthesis kernel, no contraction multiply-adds", 1, 1),
                ("synthesis kernel, the contraction's multiply-adds as 4x4x1 matrix instructions", 1, 2)]
    for name, direction, probe in variants:
        def run():
            _hip.check(P.s2cnn_so3_fft64_probe(_hip.ptr(x), _hip.ptr(y), _hip.ptr(packed[direction]), _hip.ptr(ws), ws.numel(), nvol,
                                               direction, probe, _hip.stream_ptr()))
        if direction == 1:
            PSO3.so3_rifft(spec)                      # leaves the records of a real spectrum in the workspace
        for _ in range(2):
            run()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            run()
        e1.record()
        torch.cuda.synchronize()
        out[name] = round(e0.elapsed_time(e1) / reps * 1e3, 1)
    kt = _hip.KernelTimer()
    with kt:
        for _ in range(reps):
            PSO3.so3_rifft(PSO3.so3_rfft(x))
        torch.cuda.synchronize()
    full = {k: sum(v) / len(v) * 1e3 for k, v in kt.summary().items()}
    out["analysis, whole transform"] = round(full["s2cnn_so3_analysis"], 1)
    out["synthesis, whole transform"] = round(full["s2cnn_so3_synthesis"], 1)
    bytes_dir = so3_fft_bytes(b, b, nvol)
    rows_a = full["s2cnn_so3_analysis"] - out["analysis kernel"]
    rows_s = full["s2cnn_so3_synthesis"] - out["synthesis kernel"]
    floor_us = (out["analysis kernel, no contraction and no table loads"] + rows_a) + (out["synthesis kernel, no contraction multiply-adds"] + rows_s)
    return {"workload": "per-volume kernels of the 64^3 grid, %d volumes (benchmark config 2), microseconds per launch" % nvol,
            "us": out,
            "round_trip_without_contraction_us": round(floor_us, 1),
            "frac_of_hbm_peak_without_contraction": round(2 * bytes_dir / (floor_us * 1e-6) / 1e9 / PEAK_HBM_GBS, 4),
            "frac_of_hbm_peak_shipped": round(2 * bytes_dir / ((full["s2cnn_so3_analysis"] + full["s2cnn_so3_synthesis"]) * 1e-6) / 1e9 / PEAK_HBM_GBS, 4)}


def measure_example_network(torch, name, steps, warmup, batch=32):
    """One of the reference's example networks (examples/mnist/run.py:55-98, examples/shrec17/model.py, model_original.py) in
    its training step (forward, loss, backward, SGD with momentum) on a fixed synthetic batch; time inside library calls
    listed beside the step time."""
    from s2cnn_amd import _hip, harness
    if name == "shrec17_original":
        batch = 16
    model, losses, ms = harness.train_steps(name, batch=batch, steps=steps, warmup=warmup, lr=0.01)
    with _hip.KernelTimer() as kt:
        harness.train_steps(name, batch=batch, steps=1, warmup=0, lr=0.01, model=model)
        torch.cuda.synchronize()
    calls = {k: round(sum(v), 3) for k, v in sorted(kt.summary().items(), key=lambda kv: -sum(kv[1]))}
    out = {"workload": "%s training step (s2cnn_amd/harness.py), batch %d, synthetic data" % (name, batch),
           "ms_per_step": round(ms, 3), "samples_per_s": round(batch / (ms * 1e-3), 1), "first_loss": round(losses[0], 4),
           "last_loss": round(losses[-1], 4), "library_ms": round(sum(calls.values()), 3), "library_calls_ms": calls}
    if name == "mnist":
        # the same step captured into one HIP graph and replayed (the eager step is bound by its launches)
        _, rlosses, rms = harness.train_steps_replayed(name, batch=batch, steps=max(steps, 20), warmup=3, lr=0.01)
        out["graph_replay"] = {"ms_per_step": round(rms, 3), "samples_per_s": round(batch / (rms * 1e-3), 1),
                               "first_loss": round(rlosses[0], 4), "last_loss": round(rlosses[-1], 4)}
    if name.startswith("shrec17"):
        # the same network with its BatchNorm3d + ReLU pairs evaluated inside the neighbouring transforms (same function)
        del model
        torch.cuda.empty_cache()
        torch.manual_seed(0)
        fused = harness.NETWORKS[name][0]()
        fused.fused_norm = True
        model, flosses, fms = harness.train_steps(name, batch=batch, steps=steps, warmup=warmup, lr=0.01, model=fused)
        with _hip.KernelTimer() as kt:
            harness.train_steps(name, batch=batch, steps=1, warmup=0, lr=0.01, model=model)
            torch.cuda.synchronize()
        fcalls = {k: round(sum(v), 3) for k, v in sorted(kt.summary().items(), key=lambda kv: -sum(kv[1]))}
        out["fused_norm"] = {"ms_per_step": round(fms, 3), "samples_per_s": round(batch / (fms * 1e-3), 1),
                             "first_loss": round(flosses[0], 4), "last_loss": round(flosses[-1], 4),
                             "library_ms": round(sum(fcalls.values()), 3), "library_calls_ms": fcalls}
        # ... and that step captured into one HIP graph and replayed
        del model
        torch.cuda.empty_cache()
        torch.manual_seed(0)
        fused = harness.NETWORKS[name][0]()
        fused.fused_norm = True
        _, rlosses, rms = harness.train_steps_replayed(name, batch=batch, steps=steps, warmup=3, lr=0.01, model=fused)
        out["fused_norm"]["graph_replay"] = {"ms_per_step": round(rms, 3), "samples_per_s": round(batch / (rms * 1e-3), 1),
                                             "last_loss": round(rlosses[-1], 4)}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-fft", action="store_true", help="skip the standalone FFT round trip")
    ap.add_argument("--no-mm", action="store_true", help="skip the standalone complex so3_mm (benchmark config 3)")
    ap.add_argument("--no-networks", action="store_true", help="skip benchmark configs 1 and 5 (the `config1` and `config5` objects)")
    ap.add_argument("--complex-product", action="store_true",
                    help="multiply complex spectra as the reference does instead of real-basis ones")
    ap.add_argument("--rows", action="store_true", help="also time every other op of the path (adds a `rows` object)")
    ap.add_argument("--floor", action="store_true",
                    help="also time the per-volume 64^3 kernels with their Wigner contraction compiled out (adds a `fft_floor` object)")
    ap.add_argument("--overlap", action="store_true",
                    help="also time a transform and a product of half the layer's batch on one stream and on two (adds an `overlap` object)")
    ap.add_argument("--network", nargs="?", const="config5", default=None, choices=["config5", "mnist", "shrec17", "shrec17_original"],
                    help="also time a whole network, forward + backward (adds a `network` object): config5 = the SHREC17-shaped "
                         "network of benchmark config 5 (default); mnist, shrec17, shrec17_original = the reference's example "
                         "networks (s2cnn_amd/harness.py) in a training step with SGD on a synthetic batch of 32")
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--b", type=int, default=32)
    ap.add_argument("--features", type=int, default=64)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives exist on this path); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch

    import s2cnn_amd
    from s2cnn_amd import _hip
    from s2cnn_amd.soft import so3_fft as PSO3

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    _hip.lib()
    dev = torch.device("cuda:0")
    B, F, b = args.batch, args.features, args.b
    grid = s2cnn_amd.so3_near_identity_grid()            # 3 * 8 * 8 = 192 points
    gen = torch.Generator().manual_seed(6)
    x_cpu = torch.randn(B, F, 2 * b, 2 * b, 2 * b, generator=gen)
    k_cpu = torch.randn(F, F, len(grid), generator=torch.Generator().manual_seed(7)) * math.sqrt(2.0 / (F * len(grid)))
    layer = s2cnn_amd.SO3Convolution(F, F, b, b, grid)
    layer.real_basis = not args.complex_product
    with torch.no_grad():
        layer.kernel.copy_(k_cpu)
    layer = layer.to(dev)
    x = x_cpu.to(dev).requires_grad_()

    def step():
        layer.zero_grad(set_to_none=True)
        x.grad = None
        out = layer(x)
        sum_of_squares(out).backward()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer = _hip.KernelTimer()
    t0 = time.perf_counter()
    with timer:
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    value = B / (ms_per_step * 1e-3)

    per_call = {k: sum(v) / len(v) for k, v in timer.summary().items()}
    mm_names = [n for n in per_call if n.startswith("s2cnn_so3_mm_")]   # fwd / gradx / grady of the product the layer ran
    dominant = max(mm_names, key=lambda n: per_call[n])
    flops_of = {n: mm_flops(b, B, F, F, real="_real_" in n) for n in mm_names}
    flops = flops_of[dominant]
    ach = flops / (per_call[dominant] * 1e-3) / 1e12
    roofline = {"bound": "mfma", "kernel": dominant, "achieved": round(ach, 2), "peak": PEAK_FP32_MFMA_TFLOPS,
                "unit": "TFLOP/s", "frac": round(ach / PEAK_FP32_MFMA_TFLOPS, 4),
                "traffic": MM_TRAFFIC_BYTES.get(dominant) if (B, F, b) == (16, 64, 32) else None,
                "traffic_source": "profiles/so3_mm_real_b32_B16_F64_hbm_traffic.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of "
                                  "this workload; not re-measured in this run)",
                "flop_per_launch": flops, "ms_per_launch": round(per_call[dominant], 3)}
    if "_real_" not in dominant:   # three real products per complex one: the matrix cores execute 3/4 of the algorithmic flops
        roofline["algorithmic_frac"] = roofline["frac"]
        roofline["achieved"] = round(0.75 * ach, 2)
        roofline["frac"] = round(0.75 * roofline["frac"], 4)
        roofline["flop_per_launch"] = 0.75 * flops
    kernels = {n: {"ms": round(ms, 3)} for n, ms in per_call.items()}
    for n in mm_names:
        kernels[n]["tflops"] = round(flops_of[n] / (per_call[n] * 1e-3) / 1e12, 2)
    for n in per_call:   # transforms of the step: grid bytes + spectrum bytes (half of them in the real basis)
        if n.startswith(("s2cnn_so3_analysis", "s2cnn_so3_synthesis")):
            nbytes = so3_fft_bytes(b, b, B * F) - (4 * nspec(b) * B * F if n.endswith("_real_basis") else 0)
            kernels[n]["gbs"] = round(nbytes / (per_call[n] * 1e-3) / 1e9, 1)

    # where the step goes: the library's calls (the layer), the loss of the benchmark configuration (the harness's own two
    # passes over the output) and what is left (the two small library GEMMs of the kernel spectrum, launches, gaps)
    sums = {k: sum(v) / args.steps for k, v in timer.summary().items()}
    library_ms = sum(v for k, v in sums.items() if k.startswith("s2cnn_"))
    loss_ms = sum(v for k, v in sums.items() if k.startswith("harness_loss"))
    breakdown = {"library_calls_ms": round(library_ms, 3), "harness_loss_ms": round(loss_ms, 3),
                 "other_ms": round(ms_per_step - library_ms - loss_ms, 3),
                 "layer_share_of_step": round(1.0 - loss_ms / ms_per_step, 4),
                 "samples_per_s_without_harness_loss": round(B / ((ms_per_step - loss_ms) * 1e-3), 1)}

    result = {
        "metric": "SO3Conv fwd+bwd samples/s (b=32, 64->64 ch); SO(3) FFT achieved HBM GB/s",
        "value": round(value, 2), "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "SO3Convolution fwd+bwd, batch %d, %d->%d features, b_in=b_out=%d, 192-point "
                               "near-identity grid, loss=sum(out^2) (benchmark config 4)" % (B, F, F, b)},
        "roofline": roofline, "step_breakdown": breakdown, "kernels": kernels,
    }

    # ---- standalone SO(3) FFT round trip (benchmark config 2: [256, 64, 64, 64] -> [43680, 256, 2] -> back)
    if not args.no_fft:
        del x, layer
        torch.cuda.empty_cache()
        n_fft = 256
        xf = torch.randn(n_fft, 2 * b, 2 * b, 2 * b, generator=torch.Generator().manual_seed(2)).to(dev)
        for _ in range(2):
            PSO3.so3_rifft(PSO3.so3_rfft(xf))
        torch.cuda.synchronize()
        ft = _hip.KernelTimer()
        with ft:
            for _ in range(10):
                PSO3.so3_rifft(PSO3.so3_rfft(xf))
            torch.cuda.synchronize()
        pc = {k: sum(v) / len(v) for k, v in ft.summary().items()}
        bytes_dir = so3_fft_bytes(b, b, n_fft)
        rt_ms = pc["s2cnn_so3_analysis"] + pc["s2cnn_so3_synthesis"]
        gbs = 2 * bytes_dir / (rt_ms * 1e-3) / 1e9
        result["so3_fft"] = {"workload": "SO3_fft_real -> SO3_ifft_real, [256,64,64,64] fp32 (benchmark config 2)",
                             "bound": "hbm", "bytes_round_trip": 2 * bytes_dir, "ms_round_trip": round(rt_ms, 4),
                             "analysis_ms": round(pc["s2cnn_so3_analysis"], 4), "synthesis_ms": round(pc["s2cnn_so3_synthesis"], 4),
                             "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4)}
        del xf
        torch.cuda.empty_cache()

    if not args.no_mm:
        result["so3_mm"] = measure_so3_mm(torch, dev)
    if not args.no_networks:
        result["config1"] = measure_config1(torch, dev)
        if args.network != "config5":
            result["config5"] = measure_network(torch, dev, min(args.steps, 5), 2, separate_relu=False)
    if args.rows:
        result["rows"] = measure_rows(torch, dev, not args.no_cpu)
    if args.floor:
        result["fft_floor"] = measure_fft_floor(torch, dev)
    if args.overlap:
        result["overlap"] = measure_overlap(torch, dev)
    if args.network == "config5":
        result["network"] = measure_network(torch, dev, args.steps, args.warmup)
    elif args.network:
        result["network"] = measure_example_network(torch, args.network, args.steps, args.warmup)

    # ---- CPU baseline: the oracle (a restatement of the reference's CPU branches) on a bounded sample
    if not args.no_cpu:
        from oracle import cpu_path as O
        cores = os.cpu_count() or 1
        env = os.environ.get("OMP_NUM_THREADS")
        if env:
            cores = min(cores, int(env))
        torch.set_num_threads(cores)
        Bc = 1                                           # one sample of the batch of 16
        xc = x_cpu[:Bc].clone().requires_grad_()
        kc = k_cpu.clone().requires_grad_()
        bc = torch.zeros(1, F, 1, 1, 1, requires_grad=True)
        O.so3_table(b, b, True), O.so3_table(b, b, False), O._so3_ft_matrix64(b, grid)   # tables are setup, not timed

        def cpu_step():
            xc.grad = kc.grad = bc.grad = None
            out = O.so3_conv(xc, kc, bc, b, b, grid)
            sum_of_squares(out).backward()

        cpu_step()                                       # warm-up: autograd graph, allocator, thread pool
        reps = []
        for _ in range(3):
            c0 = time.perf_counter()
            cpu_step()
            reps.append(time.perf_counter() - c0)
        med = sorted(reps)[1]
        result["cpu_baseline"] = {"value": round(Bc / med, 4), "unit": "samples/s", "cores": cores, "kind": "port",
                                  "sample": "same layer and sizes at batch %d of %d, fwd+bwd, fp32, torch threads = %d: one warm-up, "
                                            "then 3 repetitions of %s s, median taken"
                                            % (Bc, B, cores, " / ".join("%.1f" % r for r in reps))}

    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
