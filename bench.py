#!/usr/bin/env python3
"""Headline benchmark: bf16 GEMM at 8192^3 on one MI355X, plus the other benchmark configurations
as `extras`, the MFMA roofline of the dominant kernel and the CPU host-path baseline.

    python bench.py --gpus 1 --steps K --warmup W

A step is one pass of the hot path (one GEMM launch) over operands already resident in
HBM.  Prints ONE JSON line on stdout.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_F32_TFLOPS = 157.3     # MI355X f32 matrix
PEAK_HBM_GBS = 8000.0
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "gemm_bf16_8192_hbm_counters.md")


def recorded_traffic_bytes():
    """FETCH_SIZE + WRITE_SIZE per launch of the headline kernel, from the counter summary kept under profiles/
    (its line `traffic_bytes_per_launch: N`); None when the summary is absent.  Counters cannot be read inside
    this run: they come from two separate profiler passes over this same command."""
    try:
        for line in open(TRAFFIC_SUMMARY):
            if line.strip().startswith("traffic_bytes_per_launch:"):
                return float(line.split(":", 1)[1].split()[0])
    except OSError:
        pass
    return None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class Timer:
    """HIP events on the library's stream, through the C ABI."""

    def __init__(self, ag):
        self.ag = ag
        self.e0, self.e1 = C.c_void_p(), C.c_void_p()
        ag._ffi.check(ag.lib.agh_event_create(C.byref(self.e0)))
        ag._ffi.check(ag.lib.agh_event_create(C.byref(self.e1)))

    def time(self, fn, steps, warmup):
        """Returns (wall ms per step, device ms per launch)."""
        ag = self.ag
        for _ in range(warmup):
            fn()
        ag._ffi.check(ag.lib.agh_sync())
        t0 = time.perf_counter()
        ag._ffi.check(ag.lib.agh_event_record(self.e0))
        for _ in range(steps):
            fn()
        ag._ffi.check(ag.lib.agh_event_record(self.e1))
        ag._ffi.check(ag.lib.agh_sync())
        wall = (time.perf_counter() - t0) * 1e3 / steps
        ms = C.c_float()
        ag._ffi.check(ag.lib.agh_event_elapsed_ms(self.e0, self.e1, C.byref(ms)))
        return wall, ms.value / steps


def f32_to_bf16(x):
    """Round to nearest even on the bit pattern (finite synthetic data only: no NaN handling needed)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)


def rand_bf16(rng, shape, std=0.02):
    out = np.empty(shape, dtype=np.uint16)
    rows = shape[0]
    step = max(1, (1 << 24) // max(1, int(np.prod(shape[1:]))))
    for r in range(0, rows, step):  # chunked: keeps the f32 temporaries small
        out[r:r + step] = f32_to_bf16(rng.standard_normal((min(step, rows - r),) + tuple(shape[1:]), dtype=np.float32) * np.float32(std))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-extras", action="store_true", help="only the headline GEMM")
    ap.add_argument("--no-graph", action="store_true",
                    help="LeNet5 sections: time eager launches only, no graph capture / replay (replaying a captured graph "
                         "under rocprofv3 has ended in a segmentation fault inside the profiler on this image)")
    ap.add_argument("--sections", default="kernels,lenet,train",
                    help="which extras to run: kernels (other GEMMs, im2col/col2im/pool), lenet (inference), "
                         "train (training step); the last two replay captured graphs")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--settle-ms", type=float, default=200.0,
                    help="untimed repetition of the headline launch before the warm-up steps, in milliseconds")
    ap.add_argument("--calib", action="store_true",
                    help="also run a plain elementwise pass of known size (agh_relu_f32 over 2^28 floats: 1 GiB read, "
                         "1 GiB written) so HBM byte counters of a profiler run can be scaled against it")
    args = ap.parse_args()
    sections = set(args.sections.split(","))
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (--gpus 1); nothing here runs across GPUs")

    import autograph_amd as ag
    import autograph_amd._ffi  # noqa: F401
    import oracle as orc  # cpu_baseline legs only

    dev = ag.Device(0)
    info = dev.info()
    log("device:", info)
    timer = Timer(ag)
    rng = np.random.default_rng(2024)
    extras = {}

    # ---------------- headline: bf16 GEMM 8192^3, f32 accumulate, bf16 out ----------------
    n = 8192
    a = ag.Tensor.from_array(rand_bf16(rng, (n, n)))
    b = ag.Tensor.from_array(rand_bf16(rng, (n, n)))
    c = ag.Tensor.uninit((n, n), "bf16")
    # Settle: the part's clocks and power state depend on the last few hundred milliseconds; a fixed handful of
    # warm-up launches (a few ms) leaves the first timed launches on a ramp.  The same launch is repeated for
    # args.settle_ms before the W warm-up steps; none of it is inside the timed region.
    t_settle = time.perf_counter()
    settle_launches = 0
    while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
        for _ in range(8):
            ag.gemm(1.0, a, b, 0.0, c)
        ag._ffi.check(ag.lib.agh_sync())
        settle_launches += 8
    wall_ms, dev_ms = timer.time(lambda: ag.gemm(1.0, a, b, 0.0, c), args.steps, args.warmup)
    flop = 2.0 * n * n * n
    value = flop / (wall_ms * 1e-3) / 1e12
    achieved = flop / (dev_ms * 1e-3) / 1e12
    roofline = {"bound": "mfma", "kernel": "gemm_bf16_dl_kernel<256,256,2,2,1,0,true,2> (v_mfma_f32_16x16x32_bf16, direct-to-LDS loads)",
                "achieved": round(achieved, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                # HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE counter runs recorded under profiles/
                # (scaled by a copy pass of known size); refreshed whenever the kernel changes
                "traffic": recorded_traffic_bytes(),
                "algorithmic_flop_per_launch": flop, "avg_launch_ms": round(dev_ms, 4),
                "settle_ms_before_warmup": args.settle_ms, "settle_launches": settle_launches}
    log(f"bf16 gemm 8192^3: {dev_ms:.3f} ms/launch  {achieved:.1f} TFLOP/s ({100 * achieved / PEAK_BF16_TFLOPS:.1f}% of peak)")
    del c

    if args.calib:
        # ceilings measured with the same stream and events as everything else (benchlib/, a library of its own)
        import benchlib as cal
        cstream = ag.lib.agh_stream()
        sink = ag.Tensor.zeros((256,), "f32")
        blocks = 1024
        for shape, sname, iters in ((1, "16x16x32", 4096), (0, "32x32x16", 8192)):
            mflop = 2.0 * 32 * 32 * 16 * 16 * (1 + shape) * iters * 4 * blocks
            for zero in (1, 0):
                name = f"calib_mfma_only_bf16_{sname}_" + ("zero_operands" if zero else "n002_operands")
                fn = lambda: cal.check(cal.lib.calib_mfma_bf16(cstream, sink._ptr(), zero, iters, blocks, shape))  # noqa: E731
                for _ in range(40):  # ~100 ms: let the clocks settle on this load
                    fn()
                _, ms = timer.time(fn, 20, 5)
                extras[name] = {"ms": round(ms, 4), "rate": round(mflop / ms / 1e9, 1), "unit": "TFLOP/s",
                                "frac_of_peak": round(mflop / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}
                log(f"{name}: {ms:.3f} ms  {mflop / ms / 1e9:.0f} TFLOP/s")
        # the same MFMA stream (zero operands: full clock) with direct-to-LDS loads between the MFMAs, one workgroup per CU
        # cycling through a window of its own: 64 KiB windows stay in L2, 512 KiB ones come from the last-level cache,
        # 4 MiB ones from HBM.  The 256x256 GEMM tile needs 4 loads per 16 MFMAs per wave.
        dsrc_bytes = (1 << 30) + (1 << 20)
        dsrc = ag.Tensor.zeros((dsrc_bytes // 4,), "f32")
        d_iters, d_blocks = 4096, 256
        dflop = 2.0 * 32 * 32 * 16 * 16 * d_iters * 4 * d_blocks
        for window, wname in ((64 << 10, "L2"), (512 << 10, "LLC"), (4 << 20, "HBM")):
            for nld in (0, 2, 4, 8):
                if nld == 0 and wname != "L2":
                    continue
                fn = lambda: cal.check(cal.lib.calib_mfma_dma(cstream, dsrc._ptr(), dsrc_bytes, sink._ptr(), nld, window, d_iters, d_blocks))  # noqa: E731
                _, ms = timer.time(fn, 10, 3)
                fill = d_blocks * d_iters * 4.0 * nld * 1024
                extras[f"calib_mfma_dma_{nld}_loads_per_16_mfma_window_{wname}"] = {
                    "ms": round(ms, 4), "rate": round(dflop / ms / 1e9, 1), "unit": "TFLOP/s", "fill_GBps": round(fill / ms / 1e6, 1),
                    "fill_GBps_per_cu": round(fill / ms / 1e6 / d_blocks, 2)}
                log(f"MFMA + {nld} direct loads per 16 MFMAs, windows in {wname}: {ms:.3f} ms  {dflop / ms / 1e9:.0f} TFLOP/s, "
                    f"{fill / ms / 1e6:.0f} GB/s through the L1s ({fill / ms / 1e6 / d_blocks:.1f} per CU)")
        del dsrc
        nbytes = 1 << 30
        cx, cy = ag.Tensor.zeros((nbytes // 4,), "f32"), ag.Tensor.uninit((nbytes // 4,), "f32")
        for grid in (1024, 2048, 4096, 8192, 16384, 65536):
            _, ms = timer.time(lambda: cal.check(cal.lib.calib_copy(cstream, cx._ptr(), cy._ptr(), nbytes, grid)), 10, 3)
            extras[f"calib_copy_1GiB_grid{grid}"] = {"ms": round(ms, 4), "rate": round(2.0 * nbytes / ms / 1e6, 1), "unit": "GB/s",
                                                     "bytes_read": nbytes, "bytes_written": nbytes}
            log(f"copy 1 GiB, grid {grid}: {ms:.3f} ms  {2.0 * nbytes / ms / 1e6:.0f} GB/s (read + write)")
            _, ms = timer.time(lambda: cal.check(cal.lib.calib_read(cstream, cx._ptr(), sink._ptr(), nbytes, grid)), 10, 3)
            extras[f"calib_read_1GiB_grid{grid}"] = {"ms": round(ms, 4), "rate": round(nbytes / ms / 1e6, 1), "unit": "GB/s"}
            log(f"read 1 GiB, grid {grid}: {ms:.3f} ms  {nbytes / ms / 1e6:.0f} GB/s")
        del cx, cy
        # the 9:1 read:write mix of col2im at the 256x64x56x56 3x3 case, in its simplest form: 9 coalesced streams in, one out
        for dt, es in (("f32", 4), ("bf16", 2)):
            wbytes = 256 * 64 * 56 * 56 * es
            mx, my = ag.Tensor.zeros((9 * wbytes // 4,), "f32"), ag.Tensor.uninit((wbytes // 4,), "f32")
            for grid in (2048, 8192):
                _, ms = timer.time(lambda: cal.check(cal.lib.calib_mix(cstream, mx._ptr(), my._ptr(), wbytes, 9, grid)), 10, 3)
                extras[f"calib_mix_9to1_{dt}_sized_grid{grid}"] = {"ms": round(ms, 4), "rate": round(10.0 * wbytes / ms / 1e6, 1), "unit": "GB/s",
                                                                  "bytes_read": 9 * wbytes, "bytes_written": wbytes}
                log(f"9 reads : 1 write, {wbytes >> 20} MiB written ({dt} col2im size), grid {grid}: {ms:.3f} ms  {10.0 * wbytes / ms / 1e6:.0f} GB/s (read + write)")
            del mx, my
        del sink

    if not args.no_extras and "kernels" in sections:
        ks, kw = max(3, args.steps // 4), 2

        def run(name, fn, work, unit, peak, steps=ks, hbm_bytes=None):
            try:
                # the same untimed settle as the headline, shorter: clocks follow the load of the last ~50 ms
                t_s = time.perf_counter()
                while (time.perf_counter() - t_s) * 1e3 < args.settle_ms / 4:
                    fn()
                    ag._ffi.check(ag.lib.agh_sync())
                _, ms = timer.time(fn, steps, kw)
                rate = work / (ms * 1e-3) / (1e12 if unit == "TFLOP/s" else 1e9)
                extras[name] = {"ms": round(ms, 4), "rate": round(rate, 2), "unit": unit, "frac_of_peak": round(rate / peak, 4)}
                note = ""
                if hbm_bytes is not None:  # a launch that may be bound by its operand bytes rather than by its flop
                    gbs = hbm_bytes / (ms * 1e-3) / 1e9
                    extras[name].update({"algorithmic_bytes": int(hbm_bytes), "hbm_GBps": round(gbs, 1),
                                         "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 4)})
                    note = f"; {gbs:.0f} GB/s of operand bytes ({100 * gbs / PEAK_HBM_GBS:.1f}% of HBM peak)"
                log(f"{name}: {ms:.3f} ms  {rate:.1f} {unit} ({100 * rate / peak:.1f}%){note}")
            except Exception as e:  # an extra must not lose the headline line
                extras[name] = {"error": str(e)}
                log(f"{name}: FAILED {e}")

        # bf16 A^T*B / A*B^T at 8192^3 (same operands, transposed views)
        c = ag.Tensor.uninit((n, n), "bf16")
        run("gemm_bf16_8192_tn", lambda: ag.gemm(1.0, a.t(), b, 0.0, c), flop, "TFLOP/s", PEAK_BF16_TFLOPS)
        run("gemm_bf16_8192_nt", lambda: ag.gemm(1.0, a, b.t(), 0.0, c), flop, "TFLOP/s", PEAK_BF16_TFLOPS)
        # the same launch on all-zero operands: identical instruction stream, but the matrix pipes draw less
        # power, so the clocks stay up; the gap to the figure above is power management, not the schedule
        za, zb = ag.Tensor.zeros((n, n), "bf16"), ag.Tensor.zeros((n, n), "bf16")
        run("gemm_bf16_8192_zero_operands", lambda: ag.gemm(1.0, za, zb, 0.0, c), flop, "TFLOP/s", PEAK_BF16_TFLOPS)
        del za, zb
        del c
        # Dense-shaped bf16: 16384 x 4096 x 4096 with fused bias + ReLU
        xd = ag.Tensor.from_array(rand_bf16(rng, (16384, 4096)))
        wd = ag.Tensor.from_array(rand_bf16(rng, (4096, 4096)))
        bd = ag.Tensor.from_array(rand_bf16(rng, (4096,)))
        yd = ag.Tensor.uninit((16384, 4096), "bf16")
        run("dense_bf16_16384x4096x4096_bias_relu", lambda: ag.gemm(1.0, xd, wd, 0.0, yd, bias=bd, relu=True),
            2.0 * 16384 * 4096 * 4096, "TFLOP/s", PEAK_BF16_TFLOPS)
        del xd, wd, bd, yd, a, b

        def bound_gemm(dt, ta, tb, tc):
            """The C entry point with its arguments converted once, as a compiled caller holds them: for launches of a
            few microseconds the timed region is then the library call, not this script's argument handling."""
            fn_g = getattr(ag.lib, f"agh_gemm_{dt}")
            (m_, k_), n_ = ta.shape, tb.shape[1]
            cargs = [C.c_int64(m_), C.c_int64(k_), C.c_int64(n_), C.c_float(1.0), C.c_void_p(ta._ptr()), C.c_int64(ta.offset),
                     C.c_int64(ta.strides[0]), C.c_int64(ta.strides[1]), C.c_void_p(tb._ptr()), C.c_int64(tb.offset),
                     C.c_int64(tb.strides[0]), C.c_int64(tb.strides[1]), C.c_float(0.0), C.c_void_p(tc._ptr()), C.c_int64(tc.offset),
                     C.c_int64(tc.strides[0]), C.c_int64(tc.strides[1])]

            def call():
                rc = fn_g(*cargs)
                if rc:
                    ag._ffi.check(rc)
            return call

        # small, mid-size and skinny bf16 products (64 x 64 and 128 x 128 direct-to-LDS tiles, split-K for the skinny ones)
        for (m_, k_, n_) in ((1024, 1024, 1024), (2048, 2048, 2048), (4096, 4096, 4096), (16, 4096, 4096), (128, 4096, 4096)):
            sa = ag.Tensor.from_array(rand_bf16(rng, (m_, k_)))
            sb = ag.Tensor.from_array(rand_bf16(rng, (k_, n_)))
            sc = ag.Tensor.uninit((m_, n_), "bf16")
            nm = f"gemm_bf16_{m_}" if m_ == k_ == n_ else f"gemm_bf16_{m_}x{k_}x{n_}"
            run(nm, bound_gemm("bf16", sa, sb, sc), 2.0 * m_ * k_ * n_, "TFLOP/s", PEAK_BF16_TFLOPS, steps=max(ks, 50))
            del sa, sb, sc

        # f32 GEMMs: 1024, 4096 (+ transposed variants), 8192
        for sz in (1024, 4096, 8192):
            af = ag.Tensor.from_array(rng.uniform(-1, 1, (sz, sz)).astype(np.float32))
            bf = ag.Tensor.from_array(rng.uniform(-1, 1, (sz, sz)).astype(np.float32))
            cf = ag.Tensor.uninit((sz, sz), "f32")
            w = 2.0 * sz ** 3
            run(f"gemm_f32_{sz}", bound_gemm("f32", af, bf, cf), w, "TFLOP/s", PEAK_F32_TFLOPS, steps=max(ks, 50) if sz == 1024 else ks)
            if sz == 4096:
                run("gemm_f32_4096_tn", lambda: ag.gemm(1.0, af.t(), bf, 0.0, cf), w, "TFLOP/s", PEAK_F32_TFLOPS)
                run("gemm_f32_4096_nt", lambda: ag.gemm(1.0, af, bf.t(), 0.0, cf), w, "TFLOP/s", PEAK_F32_TFLOPS)
            del af, bf, cf

        # Conv2 config: im2col / col2im / conv gemm, batch 256, 64->128 ch, 56x56, 3x3 s1 p1
        bs, ci, co, hw = 256, 64, 128, 56
        for dt, es in (("f32", 4), ("bf16", 2)):
            if dt == "f32":
                x = ag.Tensor.from_array(rng.standard_normal((bs, ci, hw, hw), dtype=np.float32))
                wt = ag.Tensor.from_array((rng.standard_normal((co, ci * 9), dtype=np.float32) * np.float32(np.sqrt(2.0 / 576))))
            else:
                x = ag.Tensor.from_array(rand_bf16(rng, (bs, ci, hw, hw), 1.0))
                wt = ag.Tensor.from_array(rand_bf16(rng, (co, ci * 9), np.sqrt(2.0 / 576)))
            opts = ag.Im2ColConv2Options(filter=(3, 3), padding=(1, 1))
            cols = ag.Tensor.uninit((bs * hw * hw, ci * 9), dt)
            fn_i = getattr(ag.lib, f"agh_im2col_conv2_{dt}")
            fn_c = getattr(ag.lib, f"agh_col2im_conv2_{dt}")
            bytes_ = es * (bs * ci * hw * hw + bs * hw * hw * ci * 9)
            run(f"im2col_{dt}_conv3x3_b256", lambda: ag._ffi.check(fn_i(x._ptr(), cols._ptr(), bs, ci, hw, hw, 3, 3, 1, 1, 1, 1, 1, 1)),
                bytes_, "GB/s", PEAK_HBM_GBS)
            y = ag.Tensor.uninit((bs * hw * hw, co), dt)
            # 802816 x 576 patch matrix in, 802816 x 128 out: 0.1 flop-seconds of bf16 MFMA work against 1.13 GB (bf16) of
            # operand bytes, so in bf16 this product is bound by HBM, not by the matrix cores
            run(f"conv_gemm_{dt}_802816x576x128", lambda: ag.gemm(1.0, cols, wt.t(), 0.0, y), 2.0 * bs * hw * hw * 576 * co,
                "TFLOP/s", PEAK_F32_TFLOPS if dt == "f32" else PEAK_BF16_TFLOPS,
                hbm_bytes=es * (bs * hw * hw * (576 + co) + 576 * co))
            del y
            # the same Conv2 forward without the patch matrix: implicit GEMM on the matrix cores, NCHW in, NCHW out
            w4 = wt.into_shape((co, ci, 3, 3))
            yc = ag.Tensor.uninit((bs, co, hw, hw), dt)
            bcv = ag.Tensor.from_array(rand_bf16(rng, (co,), 0.1) if dt == "bf16" else (rng.standard_normal(co) * 0.1).astype(np.float32))
            fn_d = getattr(ag.lib, f"agh_conv2_direct_{dt}")
            peak = PEAK_F32_TFLOPS if dt == "f32" else PEAK_BF16_TFLOPS
            run(f"conv2_forward_fused_{dt}_b256_64to128_56x56", lambda: ag._ffi.check(fn_d(
                x._ptr(), w4._ptr(), None, yc._ptr(), bs, ci, hw, hw, co, 3, 3, 1, 1, 1, 1, 1, 1, 0, 0)),
                2.0 * bs * hw * hw * 576 * co, "TFLOP/s", peak)
            run(f"conv2_forward_fused_{dt}_bias_relu", lambda: ag._ffi.check(fn_d(
                x._ptr(), w4._ptr(), bcv._ptr(), yc._ptr(), bs, ci, hw, hw, co, 3, 3, 1, 1, 1, 1, 1, 1, 1, 0)),
                2.0 * bs * hw * hw * 576 * co, "TFLOP/s", peak)
            del yc, bcv, w4
            # NHWC -> NCHW copy of the layer's activation (`permuted_axes([0,3,1,2]).to_standard_layout()`, which the
            # reference's conv2_im2col ends with): the LDS-tiled transposition in agh_assign
            nhwc, nchw = ag.Tensor.uninit((bs, hw, hw, co), dt), ag.Tensor.uninit((bs, co, hw, hw), dt)
            fn_a = getattr(ag.lib, f"agh_assign_{dt}")
            run(f"assign_nhwc_to_nchw_{dt}_256x128x56x56", lambda: ag._ffi.check(fn_a(
                nhwc._ptr(), 0, hw * hw * co, 1, hw * co, co, nchw._ptr(), 0, co * hw * hw, hw * hw, hw, 1, bs, co, hw, hw)),
                2.0 * es * bs * co * hw * hw, "GB/s", PEAK_HBM_GBS)
            del nhwc, nchw
            dx = ag.Tensor.uninit((bs, ci, hw, hw), dt)
            run(f"col2im_{dt}_conv3x3_b256", lambda: ag._ffi.check(fn_c(cols._ptr(), dx._ptr(), bs, ci, hw, hw, 3, 3, 1, 1, 1, 1, 1, 1)),
                bytes_, "GB/s", PEAK_HBM_GBS)
            # MaxPool2 2x2/2 on the conv-sized activation
            py = ag.Tensor.uninit((bs, ci, hw // 2, hw // 2), dt)
            fn_p = getattr(ag.lib, f"agh_max_pool2_{dt}")
            fn_pb = getattr(ag.lib, f"agh_max_pool2_backward_{dt}")
            nx, ny = bs * ci * hw * hw, bs * ci * (hw // 2) ** 2
            run(f"max_pool2_{dt}_b256x64x56x56", lambda: ag._ffi.check(fn_p(x._ptr(), py._ptr(), bs * ci, hw, hw, 2, 2, 2, 2)),
                es * (nx + ny), "GB/s", PEAK_HBM_GBS)
            run(f"max_pool2_backward_{dt}_b256x64x56x56", lambda: ag._ffi.check(fn_pb(dx._ptr(), py._ptr(), bs * ci, hw, hw, 2, 2, 2, 2)),
                es * (2 * nx + ny), "GB/s", PEAK_HBM_GBS)
            del x, wt, cols, dx, py

    # ---------------- LeNet5 f32 inference, batch 1000 (benchmark configuration 0) ----------------
    lenet = None
    if not args.no_extras and "lenet" in sections:
        try:
            bsl = 1000
            xl = rng.uniform(0, 1, (bsl, 1, 28, 28)).astype(np.float32)

            def he(shape, fan_in):  # Uniform(-a, a), a = sqrt(2 / fan_in)
                a_ = np.sqrt(2.0 / fan_in)
                return rng.uniform(-a_, a_, shape).astype(np.float32)

            params = [he((6, 1, 5, 5), 25), he((16, 6, 5, 5), 150), he((256, 128), 256), he((128, 84), 128),
                      he((84, 10), 84), he((10,), 84)]
            model = ag.LeNet5.from_arrays(*params)
            txl = ag.Tensor.from_array(xl)
            host = C.c_void_p()
            ag._ffi.check(ag.lib.agh_host_alloc(C.byref(host), bsl * 10 * 4))
            host2 = C.c_void_p()
            ag._ffi.check(ag.lib.agh_host_alloc(C.byref(host2), bsl * 10 * 4))
            if not args.no_graph:
                model.capture(txl, host2.value)  # layered forward (5 launches) + D2H of the logits, as one graph

            def wall(fn, nwarm=100, nrep=1000):
                for _ in range(nwarm):
                    fn()
                t0 = time.perf_counter()
                for _ in range(nrep):
                    fn()
                return (time.perf_counter() - t0) * 1e3 / nrep

            # whole network in one launch, logits written straight into pinned host memory.  The entry point and
            # its arguments are bound once, as a compiled caller would hold them: the timed region is the
            # library call and the wait, not this script's attribute lookups.
            lenet_fn, sync_fn = ag.lib.agh_lenet5_forward_f32, ag.lib.agh_sync
            lenet_args = [C.c_void_p(txl._data_ptr())] + [C.c_void_p(w.as_standard_layout()._data_ptr()) for w in (
                model.conv1.weight, model.conv2.weight, model.dense1.weight, model.dense2.weight, model.dense3.weight,
                model.dense3.bias)] + [host, C.c_int64(bsl)]

            def infer():
                rc = lenet_fn(*lenet_args)
                rc |= sync_fn()  # logits are on the host when this returns
                if rc:
                    ag._ffi.check(rc)

            def infer_graph():
                model.replay()
                ag._ffi.check(ag.lib.agh_sync())

            def pipelined(launch, nwarm=100, nrep=1000):
                """K launches back to back, one wait on each side: the way this bench times every step."""
                for _ in range(nwarm):
                    launch()
                ag._ffi.check(sync_fn())
                t0 = time.perf_counter()
                for _ in range(nrep):
                    launch()
                ag._ffi.check(sync_fn())
                return (time.perf_counter() - t0) * 1e3 / nrep

            gpu_ms = wall(infer)
            got = np.ctypeslib.as_array(C.cast(host.value, C.POINTER(C.c_float)), shape=(bsl, 10)).copy()
            gpu_pipe_ms = pipelined(lambda: lenet_fn(*lenet_args))
            if args.no_graph:
                graph_ms = graph_pipe_ms = None
            else:
                graph_ms = wall(infer_graph, 50, 300)
                graph_pipe_ms = pipelined(model.replay, 50, 300)
            _, kernel_ms = timer.time(lambda: model.forward_single_launch(txl, host.value), 50, 20)
            # layer-by-layer path (12 launches, im2col + gemm convolutions), eager, each layer allocating its output
            _, layered_ms = timer.time(lambda: model.forward(txl, algorithm="im2col"), 20, 5)
            # the same layer objects with each layer's own fused form (conv+relu+pool, dense+relu): 5 launches, eager
            _, fused_eager_ms = timer.time(lambda: model.forward_fused(txl), 20, 5)
            lenet = {"gpu_ms": round(gpu_ms, 4), "gpu_kernel_ms": round(kernel_ms, 4), "gpu_pipelined_ms": round(gpu_pipe_ms, 4),
                     "gpu_graph_5_launches_ms": None if graph_ms is None else round(graph_ms, 4),
                     "gpu_graph_5_launches_pipelined_ms": None if graph_pipe_ms is None else round(graph_pipe_ms, 4),
                     "gpu_layered_5_launches_eager_ms": round(fused_eager_ms, 4),
                     "gpu_layered_im2col_eager_ms": round(layered_ms, 4),
                     "what": "gpu_ms: one launch of the whole-network kernel (input resident in HBM, [1000,10] logits written "
                             "into pinned host memory), wall clock per inference including the host-side wait; "
                             "gpu_kernel_ms: the same launch between HIP events; gpu_pipelined_ms: 1000 such launches back to "
                             "back with one wait at the end, per launch; gpu_graph_5_launches_ms: graph replay of "
                             "conv+relu+pool x2 and 3 Dense GEMMs plus D2H through the per-layer entry points, with the "
                             "host-side wait (…_pipelined_ms: replays back to back); gpu_layered_5_launches_eager_ms: the "
                             "same five per-layer calls issued eagerly, each allocating its output; "
                             "gpu_layered_im2col_eager_ms: the 12-launch layer-by-layer path (im2col + gemm, relu, pool)"}
            if not args.no_cpu:
                thr = orc.max_threads()
                want = orc.lenet5_forward_f32(xl, *params, direct="packed")
                t0 = time.perf_counter()
                ncpu = 40
                for _ in range(ncpu):
                    orc.lenet5_forward_f32(xl, *params, direct="packed")
                cpu_ms = (time.perf_counter() - t0) * 1e3 / ncpu
                t0 = time.perf_counter()
                for _ in range(10):
                    orc.lenet5_forward_f32(xl, *params, direct=True)
                cpu_axpy_ms = (time.perf_counter() - t0) * 1e3 / 10
                lenet.update({"cpu_ms": round(cpu_ms, 3), "cpu_threads": thr, "cpu_plain_direct_conv_ms": round(cpu_axpy_ms, 3),
                              "speedup": round(cpu_ms / gpu_ms, 1),
                              "speedup_single_kernel": round(cpu_ms / gpu_ms, 1),
                              "speedup_single_kernel_pipelined": round(cpu_ms / gpu_pipe_ms, 1),
                              "speedup_api_graph": None if graph_ms is None else round(cpu_ms / graph_ms, 1),
                              "speedup_api_graph_pipelined": None if graph_pipe_ms is None else round(cpu_ms / graph_pipe_ms, 1),
                              "speedup_api_eager": round(cpu_ms / fused_eager_ms, 1),
                              "speedup_api_im2col_eager": round(cpu_ms / layered_ms, 1),
                              "max_abs_diff_vs_cpu": float(np.abs(got - want).max()),
                              "cpu_what": "oracle port of the host path: f32 convolutions packed to [f32; 8] and register-tiled as "
                                          "conv_direct (AVX2 + FMA, images dealt to all cores), relu and pooling over all cores, "
                                          "blocked sgemm on <=4 threads for Dense; cpu_plain_direct_conv_ms: the same with a plain "
                                          "axpy convolution loop"})
            extras["lenet5_f32_infer_b1000"] = lenet
            log("lenet5 f32 b=1000:", lenet)
            del model
        except Exception as e:
            extras["lenet5_f32_infer_b1000"] = {"error": str(e)}
            log("lenet5: FAILED", e)

    # ---------------- LeNet5 training step, batch 100 (benchmark configuration 4) ----------------
    if not args.no_extras and "train" in sections:
        for dt in ("bf16", "f32"):
            key = f"lenet5_{dt}_train_b100"
            try:
                bst = 100
                conv = f32_to_bf16 if dt == "bf16" else (lambda a: a)
                xt = conv(rng.uniform(0, 1, (bst, 1, 28, 28)).astype(np.float32))
                tt = rng.integers(0, 10, bst).astype(np.uint8)

                def he2(shape, fan_in):
                    a_ = np.sqrt(2.0 / fan_in)
                    return conv(rng.uniform(-a_, a_, shape).astype(np.float32))

                tparams = [he2((6, 1, 5, 5), 25), he2((16, 6, 5, 5), 150), he2((256, 128), 256), he2((128, 84), 128),
                           he2((84, 10), 84), he2((10,), 84)]
                trainer = ag.LeNet5Trainer(ag.LeNet5.from_arrays(*tparams), bst, learning_rate=0.01, optimizer=ag.SGD(0.01))
                txx = ag.Tensor.from_array(xt)
                tbuf = ag.Buffer(bst)
                ag._ffi.check(ag.lib.agh_memcpy_h2d(tbuf.ptr, tt.ctypes.data, bst))
                if not args.no_graph:
                    trainer.capture(txx, tbuf)

                def train_graph():
                    trainer.replay()
                    ag._ffi.check(ag.lib.agh_sync())  # the loss is in host memory when this returns

                def train_eager():
                    trainer.step(txx, tbuf)
                    ag._ffi.check(ag.lib.agh_sync())

                g_ms = None
                if not args.no_graph:
                    for _ in range(20):
                        train_graph()
                    t0 = time.perf_counter()
                    for _ in range(200):
                        train_graph()
                    g_ms = (time.perf_counter() - t0) * 1e3 / 200
                for _ in range(5):
                    train_eager()
                t0 = time.perf_counter()
                for _ in range(50):
                    train_eager()
                e_ms = (time.perf_counter() - t0) * 1e3 / 50
                if g_ms is None:
                    g_ms = e_ms
                rec = {"gpu_ms": round(g_ms, 4), "gpu_eager_ms": round(e_ms, 4), "last_loss": round(trainer.loss(), 4),
                       "what": "forward + summed cross-entropy + backward + SGD(momentum 0.01) update in six kernels on one stream: the forward pass, the input-gradient chain, the dense weight gradients + bias gradient + loss, the convolutions' weight gradients (per-image partial sums, then their reduction), the update; gpu_ms: "
                               "graph replay, wall clock per step including the host-side wait for the loss; "
                               "gpu_eager_ms: the same launches issued one by one from the host"}
                if not args.no_cpu:
                    orc.lenet5_train_step(xt, tt, tparams, lr=0.01, momentum=0.01)
                    t0 = time.perf_counter()
                    for _ in range(10):
                        orc.lenet5_train_step(xt, tt, tparams, lr=0.01, momentum=0.01)
                    c_ms = (time.perf_counter() - t0) * 1e3 / 10
                    rec.update({"cpu_ms": round(c_ms, 3), "speedup": round(c_ms / g_ms, 1),
                                "cpu_what": "oracle port of the host ops chained in Python; its bf16 GEMMs accumulate in f32 "
                                            "(the host's per-operation-rounded fold would be slower still)"})
                extras[key] = rec
                log(f"lenet5 {dt} train b=100:", rec)
                del trainer
            except Exception as e:
                extras[key] = {"error": str(e)}
                log(f"lenet5 {dt} train: FAILED", e)

    # ---------------- CPU baseline: the oracle's restatement of the host path ----------------
    cpu = None
    if not args.no_cpu:
        t0 = time.perf_counter()
        s = 1024  # bounded sample of the same workload: scalar bf16 fold is O(mnk) on one thread, ~11 s
        ha, hb = rand_bf16(rng, (s, s)), rand_bf16(rng, (s, s))
        t1 = time.perf_counter()
        orc.gemm_bf16_hostfold(ha, hb)
        dt_bf16 = time.perf_counter() - t1
        sf = 2048
        fa, fb = rng.uniform(-1, 1, (sf, sf)).astype(np.float32), rng.uniform(-1, 1, (sf, sf)).astype(np.float32)
        threads = min(4, orc.max_threads())
        orc.gemm_f32_host(fa[:256], fb, threads=threads)
        t1 = time.perf_counter()
        orc.gemm_f32_host(fa, fb, threads=threads)
        dt_f32 = time.perf_counter() - t1
        cpu = {"value": round(2.0 * s ** 3 / dt_bf16 / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
               "sample": f"bf16 {s}^3 GEMM, host path = scalar fold with per-op bf16 rounding, 1 thread ({dt_bf16:.2f} s); "
                         f"the 8192^3 job is the same loop x{(8192 / s) ** 3:.0f}",
               "f32_sgemm": {"value": round(2.0 * sf ** 3 / dt_f32 / 1e12, 4), "unit": "TFLOP/s", "cores": threads,
                             "sample": f"f32 {sf}^3 blocked sgemm ({dt_f32:.2f} s)"},
               "host_cores_visible": os.cpu_count()}
        log(f"cpu baseline: bf16 fold {cpu['value']} TFLOP/s (1 thread), f32 sgemm {cpu['f32_sgemm']['value']} TFLOP/s ({threads} threads), {time.perf_counter() - t0:.1f} s")

    line = {
        "metric": "bf16/f32 GEMM TFLOP/s @8192^3 (% MFMA peak); LeNet5 b=1000 infer ms",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "bf16 GEMM C=A*B, M=N=K=8192, row-major, f32 accumulate, bf16 out (BASELINE configs[2])",
                   "device": info["name"], "compute_units": info["compute_units"]},
        "roofline": roofline, "cpu_baseline": cpu, "extras": extras,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
