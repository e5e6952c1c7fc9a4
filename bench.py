#!/usr/bin/env python3
"""Benchmark of the witness-generation hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]

Prints ONE JSON line.  `value` is the int64 GEMM throughput (Gmac/s) of benchmark config 4
(512 x 7168 against W[18432,7168], config-1 operand ranges, shift 29) through the C ABI with operands
resident in HBM; one step = one call of int64_64_bmm_broadcast_launcher.  The same line carries the
other shapes the metric names (config-1 GEMM, full-range config 4, softmax / SiLU / sigmoid / RMSNorm
HBM GB/s) under "extra", the roofline of the dominant kernel (with the figures of config 1 and of the HBM-bound
shapes the metric names as flat keys inside it, and once more at the end of the line under "summary"), the calls on
operands never seen (--only cold), and a CPU baseline timed on this host.

Nothing is timed before it has been checked: the headline product is compared with torch's int64 matmul on the CPU
(same input bytes) on a block of columns before the timed loop starts, and the run aborts on a mismatch; the other
legs keep samples of their inputs and outputs, which the CPU leg compares with torch (GEMMs, einsums) or with the
scalar C restatement of the kernels (softmax, SiLU, sigmoid, RMSNorm) before the JSON line is printed.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (os.path.join(ROOT, "zk-deepseek_amd"),):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
I8_MFMA_PEAK_TOPS = 5000.0     # MI355X dense int8 MFMA


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20, help="untimed calls before the timed steps (at least; see SPIN_UP_MS)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="comma list of legs: gemm,extra,small,cold,prepared,cpu,calib (default gemm,extra,cpu; small = configs 1 and 2 of extra alone, cold = the calls on operands never seen alone, prepared = config 4 on prepared weights alone)")
    return ap.parse_args()


def randint(gen, lo, hi, shape, dtype=None):
    import torch
    return torch.randint(lo, hi, shape, generator=gen, dtype=dtype or torch.int64)


def full_range(gen, shape):
    import torch
    hi = torch.randint(-(1 << 31), 1 << 31, shape, generator=gen, dtype=torch.int64)
    lo = torch.randint(0, 1 << 32, shape, generator=gen, dtype=torch.int64)
    return (hi << 32) | lo


SPIN_UP_MS = 60.0    # an idle device needs some 40 ms of work to reach its clocks (measured: the first 50 config-4
                     # GEMM calls after a pause average 0.76 ms, every later 50 average 0.70 ms)


def spin_up(fn, at_least=0):
    """untimed calls of fn: `at_least` of them, and as many more as it takes to keep the device busy for SPIN_UP_MS"""
    import torch
    calls = at_least
    for _ in range(at_least):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < SPIN_UP_MS:
        for _ in range(4):
            fn()
        calls += 4
        torch.cuda.synchronize()
    return calls


def timed(K, fn, steps, warmup):
    """average milliseconds per call, measured with HIP events on the null stream (where the library launches)"""
    import torch
    spin_up(fn, warmup)
    K.lib.zk_timer_start()
    for _ in range(steps):
        fn()
    ms = K.lib.zk_timer_stop_ms()
    torch.cuda.synchronize()
    return ms / steps


def sample_rows(n, count, seed):
    """`count` distinct indices below n: both ends and a seeded draw"""
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    return sorted(set([0, n - 1] + torch.randint(0, n, (count,), generator=g).tolist()))


def gemm_sample(name, A, W, C, R, c, b_rs=1, rows=8, cols=96):
    """Keeps sampled rows of A, sampled rows of W and the matching block of the GPU's C (and R) on the host; returns a
    check that compares them with the 128-bit CPU restatement of the kernel (valid for every operand range)."""
    import torch
    Bd, M, Kd = A.shape
    N = W.shape[0]
    ri = torch.as_tensor(sample_rows(Bd * M, rows, 11), dtype=torch.long, device="cuda")
    ci = torch.as_tensor(sample_rows(N, cols, 13), dtype=torch.long, device="cuda")
    a = A.reshape(-1, Kd)[ri].cpu().numpy()
    w = W[ci].cpu().numpy()
    cg = C.reshape(-1, N)[ri][:, ci].cpu().numpy()
    rg = R.reshape(-1, N)[ri][:, ci].cpu().numpy() if R is not None else None

    def check(ck, np):
        ce, re_ = ck.int64_bmm_broadcast(np.ascontiguousarray(a[None]), np.ascontiguousarray(w), 1, b_rs, c)
        if not np.array_equal(ce[0], cg) or (rg is not None and not np.array_equal(re_[0], rg)):
            raise Mismatch("%s: the GPU result differs from the CPU restatement on the sampled block" % name)
        return "%dx%d sampled outputs equal the 128-bit CPU restatement" % (len(ri), len(ci))
    return (name, check)


def gemm_leg(K, A, W, c, steps, warmup, samples=None, name=None, host=None):
    """times one bmm shape; before that, one call is checked: against torch's CPU int64 matmul on sampled columns when
    the host copies of the operands are given (`host`), and a sampled block is kept for the CPU leg's 128-bit check"""
    import torch
    Bd, M, Kd = A.shape
    N = W.shape[0]
    C = torch.empty((Bd, M, N), dtype=torch.int64, device="cuda")
    R = torch.empty((Bd, M, N), dtype=torch.int64, device="cuda")
    fn = K.lib.int64_64_bmm_broadcast_launcher if W.dtype == torch.int64 else K.lib.int64_32_bmm_broadcast_launcher

    def call():
        fn(A.data_ptr(), W.data_ptr(), C.data_ptr(), R.data_ptr(), 1, 1, c, Bd, M, Kd, N)

    call()
    K._check("gemm bench")
    checked = []
    if host is not None:
        cols = sample_rows(N, min(N, 128), 17)
        verify_gemm_columns(name, host[0], host[1].to(torch.int64), C, R, c, cols)
        checked.append("torch CPU int64 matmul on %d columns" % len(cols))
    if samples is not None:
        samples.append(gemm_sample(name, A, W, C, R, c))
    ms = timed(K, call, steps, warmup)
    K._check("gemm bench")
    path, la, lb = K.gemm_last_plan()
    macs = Bd * M * N * Kd
    return {"ms": ms, "gmacs": macs / ms / 1e6, "macs": macs, "path": {1: "valu", 2: "mfma_i8"}.get(path, "?"),
            "limbs_a": la, "limbs_b": lb, "digit_pairs": K.gemm_last_pairs(), "checked_before_timing": checked}


class Mismatch(Exception):
    pass


def verify_gemm_columns(name, A_h, W_h, C, R, c, cols):
    """GPU quotient and remainder of X @ W^T against torch's int64 matmul on the CPU (the reference's CPU path,
    inference/model.py:179-181) on the columns `cols`: C == product >> c and C * 2^c + R == product (wrapping).
    Valid wherever the 128-bit sum fits 64 bits, and at c == 0 for any operands."""
    import torch
    cols_t = torch.as_tensor(cols, dtype=torch.long)
    prod = torch.matmul(A_h.reshape(-1, A_h.shape[-1]), W_h[cols_t].T.contiguous())
    Cg = C.reshape(-1, C.shape[-1])[:, cols_t.cuda()].cpu()
    if not torch.equal(Cg, prod >> c):
        raise Mismatch("%s: the GPU quotient differs from torch's CPU int64 matmul >> %d" % (name, c))
    if R is not None:
        Rg = R.reshape(-1, R.shape[-1])[:, cols_t.cuda()].cpu()
        if not torch.equal((Cg << c) + Rg, prod) or bool((Rg < 0).any()) or bool((Rg >> c).any()):
            raise Mismatch("%s: C * 2^c + R does not rebuild the CPU product" % name)
    return len(cols)


def main():
    try:
        run()
    except Mismatch as e:
        print("bench.py: RESULT CHECK FAILED, nothing is reported: %s" % e, file=sys.stderr)
        sys.stdout.flush()
        sys.stderr.flush()
        os._exit(3)


def run():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives, no sharding); --gpus must be 1",
              file=sys.stderr)
        sys.exit(2)
    import torch
    import kernel as K
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    legs = set(args.only.split(",")) if args.only else {"gemm", "extra", "cpu"}
    if args.no_cpu:
        legs.discard("cpu")
    gen = torch.Generator(device="cpu").manual_seed(4000)
    extra = {}

    # ---------------- headline: config 4 GEMM ----------------------------------------------
    M, Kd, N, c = 512, 7168, 18432, 29
    A_h = randint(gen, -(1 << 20), 1 << 20, (1, M, Kd))
    W_h = randint(gen, -(1 << 16), 1 << 16, (N, Kd))
    A, W = A_h.cuda(), W_h.cuda()
    # the timed region proper: W warmup calls, then exactly K steps between synchronisations
    Cb = torch.empty((1, M, N), dtype=torch.int64, device="cuda")
    Rb = torch.empty((1, M, N), dtype=torch.int64, device="cuda")

    def step():
        K.lib.int64_64_bmm_broadcast_launcher(A.data_ptr(), W.data_ptr(), Cb.data_ptr(), Rb.data_ptr(),
                                              1, 1, c, 1, M, Kd, N)

    # checked before anything is timed: 128 columns (both ends and a seeded draw) against torch on the CPU
    step()
    gcols = torch.Generator(device="cpu").manual_seed(4002)
    check_cols = sorted(set(list(range(32)) + list(range(N - 32, N)) + torch.randint(0, N, (64,), generator=gcols).tolist()))
    verified = {"gemm_config4": "C and C*2^c+R equal torch CPU int64 matmul on %d of %d columns, before timing"
                                % (verify_gemm_columns("config-4 GEMM", A_h, W_h, Cb, Rb, c, check_cols), N)}
    samples = []          # (name, check) pairs run by the CPU leg before anything is reported

    untimed_calls = spin_up(step, args.warmup)
    t0 = time.perf_counter()
    K.lib.zk_timer_start()
    for _ in range(args.steps):
        step()
    ev_ms = K.lib.zk_timer_stop_ms()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    K._check("config-4 GEMM")
    path, la, lb = K.gemm_last_plan()
    macs = M * N * Kd
    ms_per_step = wall_ms / args.steps
    kern_ms = ev_ms / args.steps
    value = macs / ms_per_step / 1e6                     # Gmac/s

    if path == 2:
        pairs = la * lb
        ops = 2.0 * pairs * macs                         # i8 multiply-adds issued as MFMA, counted as 2 ops
        achieved = ops / (kern_ms * 1e-3) / 1e12
        # what the i8 matrix pipe sustains on this box, measured live: register-resident and GEMM-shaped (fragments
        # from LDS + a barrier per step), with zero operands and with random bytes.  The device is power managed
        # and MFMAs on randomly toggling bytes (which the digits of real operands are) run slower than on zeros.
        probe = {}
        for name, with_lds, rnd in (("regs_zeros", 0, 0), ("regs_random", 0, 1), ("lds_zeros", 1, 0), ("lds_random", 1, 1)):
            probe[name] = K.lib.zk_probe_mfma_i8_tops(with_lds, rnd, 3000)
        K._check("MFMA probe")
        roofline = {"bound": "mfma", "achieved": achieved, "peak": I8_MFMA_PEAK_TOPS, "unit": "TOP/s",
                    "frac": achieved / I8_MFMA_PEAK_TOPS, "traffic": measured_traffic(),
                    "traffic_source": "committed rocprofv3 --pmc profile of this kernel and workload "
                                      "(profiles/gemm_config4_i8mfma_hbm_traffic.md), NOT measured in this run",
                    "path_peak_measured": probe,
                    "frac_of_measured_random_data_peak": achieved / probe["regs_random"] if probe["regs_random"] else None,
                    "note": "i8 MFMA ops = 2 * limbs_a * limbs_b * M*N*K (%dx%d limb pairs per int64 MAC); "
                            "duration = HIP events over the whole launcher; path_peak_measured = "
                            "v_mfma_i32_32x32x32_i8 microbenchmark on this device, TOP/s" % (la, lb)}
    else:
        achieved = macs / (kern_ms * 1e-3) / 1e12
        roofline = {"bound": "valu", "achieved": achieved, "peak": None, "unit": "Tmac/s", "frac": None,
                    "traffic": None, "note": "VALU 64-bit multiply-add path; no published peak"}

    launch_floor_us = None
    if legs & {"extra", "small"}:
        # what two dependent, nearly empty launches cost back to back (the shape of a split-K call: a streaming kernel
        # and a finishing kernel), measured on this device: the part of config 1's time that no kernel can remove
        launch_floor_us = K.lib.zk_probe_launch_pair_us(252, 200)
        K._check("launch pair probe")
        extra["launch_pair_252_workgroups_us"] = launch_floor_us
        # the GEMMs smaller than the device ("small" alone: the legs a kernel trace of them needs)
        # config 1 (M=16): weight-bandwidth bound
        g1 = torch.Generator(device="cpu").manual_seed(1000)
        A1_h = randint(g1, -(1 << 20), 1 << 20, (1, 16, 7168))
        W1_h = randint(g1, -(1 << 16), 1 << 16, (576, 7168))
        A1, W1 = A1_h.cuda(), W1_h.cuda()
        nm = "gemm_config1_16x7168x576"
        extra[nm] = gemm_leg(K, A1, W1, 29, 200, 20, samples, nm, host=(A1_h, W1_h))
        # config 2's GEMMs (one expert FFN at M = 128): w1/w3 [2048,7168] and w2 [7168,2048], shift 16
        g2m = torch.Generator(device="cpu").manual_seed(2000)
        X2_h = randint(g2m, -(1 << 20), 1 << 20, (1, 128, 7168))
        W21_h = randint(g2m, -(1 << 16), 1 << 16, (2048, 7168))
        H2_h = randint(g2m, -(1 << 20), 1 << 20, (1, 128, 2048))
        W22_h = randint(g2m, -(1 << 16), 1 << 16, (7168, 2048))
        X2, W21, H2, W22 = X2_h.cuda(), W21_h.cuda(), H2_h.cuda(), W22_h.cuda()
        nm = "gemm_config2_w1_128x7168x2048"
        extra[nm] = gemm_leg(K, X2, W21, 16, 100, 10, samples, nm, host=(X2_h, W21_h))
        nm = "gemm_config2_w2_128x2048x7168"
        extra[nm] = gemm_leg(K, H2, W22, 16, 100, 10, samples, nm, host=(H2_h, W22_h))
        del X2, W21, H2, W22, X2_h, W21_h, H2_h, W22_h

    if legs & {"extra", "cold"}:
        # Calls on operands the library has not seen.  The reference's driver builds every layer anew on the device for
        # every position (inference/generate.py:227-238) and loads each routed expert from disk when it is hit
        # (inference/model.py:1362-1363), so in an unchanged drop-in the weight pointers of most calls are new, or are
        # recycled addresses that hold other contents than last time.  Wall clock of ONE call from before the call to
        # after a device synchronisation (so a readback that blocks the host is inside), next to the same single call
        # on warm operands: (a) freshly allocated A and W at addresses never passed before; (b) a known address whose
        # contents were overwritten in place with wider values (W from 17 to 31 bits) since the library last saw it.
        def one_call_ms(fn):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            fn()
            t_ret = time.perf_counter()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) * 1e3, (t_ret - t0) * 1e3

        def cold_leg(name, Mc, Kc, Nc, shift):
            gc_ = torch.Generator(device="cuda").manual_seed(4100 + Mc)
            keep = []                       # everything stays allocated: no address comes back
            mk = lambda lo, hi, *shape: torch.randint(lo, hi, shape, generator=gc_, dtype=torch.int64, device="cuda")
            Cc = torch.empty((1, Mc, Nc), dtype=torch.int64, device="cuda")
            Rc = torch.empty_like(Cc)
            fn64 = K.lib.int64_64_bmm_broadcast_launcher

            def call(Ax, Wx):
                fn64(Ax.data_ptr(), Wx.data_ptr(), Cc.data_ptr(), Rc.data_ptr(), 1, 1, shift, 1, Mc, Kc, Nc)

            res = {}
            firsts, blocked = [], []
            for rep in range(3):
                Ax, Wx = mk(-(1 << 20), 1 << 20, 1, Mc, Kc), mk(-(1 << 16), 1 << 16, Nc, Kc)
                keep += [Ax, Wx]
                ms, ret = one_call_ms(lambda: call(Ax, Wx))
                firsts.append(ms)
                blocked.append(ret)
            K._check(name)
            res["first_call_new_addresses_ms"] = sorted(firsts)[1]
            res["first_call_host_blocked_ms"] = sorted(blocked)[1]
            Ax, Wx = keep[-2], keep[-1]
            for _ in range(3):
                call(Ax, Wx)
            warm = sorted(one_call_ms(lambda: call(Ax, Wx)) for _ in range(5))[2]
            res["warm_single_call_ms"], res["warm_host_blocked_ms"] = warm
            # the same addresses, wider contents written in place behind the library's back
            Wx.copy_(mk(-(1 << 30), 1 << 30, Nc, Kc))
            hits0 = K.lib.zk_gemm_guard_hits()
            ms, ret = one_call_ms(lambda: call(Ax, Wx))
            res["recycled_address_wider_contents_ms"] = ms
            res["recycled_address_host_blocked_ms"] = ret
            samples.append(gemm_sample(name + "_recycled", Ax, Wx, Cc, Rc, shift))
            ms2, _ = one_call_ms(lambda: call(Ax, Wx))
            res["call_after_that_ms"] = ms2
            res["guarded_recomputations"] = int(K.lib.zk_gemm_guard_hits() - hits0)
            K._check(name)
            res["first_over_warm"] = res["first_call_new_addresses_ms"] / res["warm_single_call_ms"]
            res["recycled_over_warm"] = res["recycled_address_wider_contents_ms"] / res["warm_single_call_ms"]
            extra[name] = res
            del keep

        cold_leg("cold_gemm_config4_512x7168x18432", 512, 7168, 18432, 29)
        cold_leg("cold_gemm_config2_w1_128x7168x2048", 128, 7168, 2048, 16)
        cold_leg("cold_gemm_config1_16x7168x576", 16, 7168, 576, 29)
        torch.cuda.empty_cache()

    if "extra" in legs:
        # config 4, full-range operands (two's-complement wraparound)
        g4 = torch.Generator(device="cpu").manual_seed(4001)
        Af_h = full_range(g4, (1, M, Kd))
        Wf_h = full_range(g4, (N, Kd))
        Af, Wf = Af_h.cuda(), Wf_h.cuda()
        nm = "gemm_config4_full_range"
        extra[nm] = gemm_leg(K, Af, Wf, 29, max(3, args.steps // 4), 1, samples, nm)
        # the same product modulo 2^64 (shift 0): only the digit pairs below 2^64 are multiplied; torch's CPU matmul wraps
        # the same way, so this variant is checked against the reference's CPU path itself
        nm = "gemm_config4_full_range_shift0"
        extra[nm] = gemm_leg(K, Af, Wf, 0, max(3, args.steps // 4), 1, samples, nm, host=(Af_h, Wf_h))
        full_range_host = (Af_h, Wf_h[:256].clone())        # the CPU leg times the reference's path on these too
        del Af, Wf, Af_h, Wf_h
        # real-model operand widths: Q31 activations (|x| < 2^37), int32 weights
        Am = randint(g4, -(1 << 37), 1 << 37, (1, M, Kd)).cuda()
        Wm = randint(g4, -(1 << 31), 1 << 31, (N, Kd)).to(torch.int32).cuda()
        nm = "gemm_config4_q31_x_int32"
        extra[nm] = gemm_leg(K, Am, Wm, 30, max(3, args.steps // 2), 1, samples, nm)
        del Am, Wm
    if legs & {"extra", "prepared"}:
        # the headline shape with the weights prepared once as digit planes (zk_gemm_prepare_weights): what a model
        # with static weights gets; the one-time preparation is timed separately and is NOT part of `value`
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        K.prepare_weights(W[0] if W.dim() == 3 else W)
        prep_ms = (time.perf_counter() - t0) * 1e3
        extra["gemm_config4_prepared_weights"] = gemm_leg(K, A, W, c, args.steps, 5, samples, "gemm_config4_prepared_weights", host=(A_h, W_h))
        extra["gemm_config4_prepared_weights"]["prepare_once_ms"] = prep_ms
        K.release_weights(W[0] if W.dim() == 3 else W)

    if "extra" in legs:
        # other instruction path on the headline shape, for the comparison
        K.lib.zk_gemm_set_path(1 if path == 2 else 2)
        extra["gemm_config4_other_path"] = gemm_leg(K, A, W, c, 3, 1, samples, "gemm_config4_other_path", host=(A_h, W_h))
        K.lib.zk_gemm_set_path(0)

        # memory-bound kernels, 16 algorithmic bytes per element
        K.softmax_init_q19()
        K.silu_init_q23()

        def hbm(name, fn, nelem, bytes_per_elem=16.0, extra_bytes=0.0, steps=30, sample=None):
            ms = timed(K, fn, steps, 3)
            K._check(name)
            gbs = (nelem * bytes_per_elem + extra_bytes) / (ms * 1e-3) / 1e9
            extra[name] = {"ms": ms, "GBps": gbs, "frac_hbm_peak": gbs / HBM_PEAK_GBS, "elements": nelem}
            if ms < 0.05 and launch_floor_us:
                # a launch this short is bound by the launch itself as much as by its bytes: next to the HBM fraction,
                # the fraction of (one launch as measured on this device + the bytes at the HBM peak)
                floor_us = launch_floor_us / 2.0 + (nelem * bytes_per_elem + extra_bytes) / (HBM_PEAK_GBS * 1e9) * 1e6
                extra[name]["one_launch_us"] = launch_floor_us / 2.0
                extra[name]["frac_of_launch_plus_hbm_floor"] = floor_us / (ms * 1e3)
            if sample is not None:
                samples.append((name, sample()))

        # samples of a leg's input and output, kept on the host for the CPU leg's comparison with the scalar restatement
        def rows_of(t, width, count, seed):
            ri = torch.as_tensor(sample_rows(t.numel() // width, count, seed), dtype=torch.long, device="cuda")
            return ri, t.reshape(-1, width)[ri].cpu().numpy()

        def softmax_sample(name, x, y, which):
            def make():
                ri, xs = rows_of(x, x.shape[-1], 48, 3)
                ys = y.reshape(-1, y.shape[-1])[ri].cpu().numpy()

                def check(ck, np):
                    got = getattr(ck, which)(np.ascontiguousarray(xs[None, None]))[0][0, 0]
                    if not np.array_equal(got, ys):
                        raise Mismatch("%s: sampled rows differ from the CPU restatement" % name)
                    return "%d sampled rows equal the CPU restatement" % len(ri)
                return check
            return make

        def act_sample(name, x, y, which):
            def make():
                ri, xs = rows_of(x, 1024, 64, 5)
                ys = y.reshape(-1, 1024)[ri].cpu().numpy()

                def check(ck, np):
                    if not np.array_equal(getattr(ck, which)(np.ascontiguousarray(xs[None])), ys[None]):
                        raise Mismatch("%s: sampled elements differ from the CPU restatement" % name)
                    return "%d sampled elements equal the CPU restatement" % xs.size
                return check
            return make

        def rms_sample(name, x, w, rms_out, y):
            def make():
                ri, xs = rows_of(x, x.shape[-1], 16, 7)
                ys = y[ri].cpu().numpy()
                rs = rms_out[ri].cpu().numpy()
                wh = w.cpu().numpy()

                def check(ck, np):
                    ce, re_ = ck.RMS_Norm_int64(np.ascontiguousarray(xs), wh, 1, x.shape[-1])
                    if not np.array_equal(ce, ys) or not np.array_equal(re_, rs):
                        raise Mismatch("%s: sampled rows differ from the CPU restatement" % name)
                    return "%d sampled rows (values and statistic) equal the CPU restatement" % len(ri)
                return check
            return make

        for S in (1024, 4096):
            g3 = torch.Generator(device="cpu").manual_seed(3000 + S)
            x = randint(g3, -(6 << 19), 6 << 19, (1, S, 128, 1024))
            if S == 1024:
                x += torch.full((S, 1024), -(64 << 36), dtype=torch.int64).triu_(1).unsqueeze(1)
            R = x.cuda()
            del x
            Cs = torch.empty_like(R)
            nm = "softmax_q19_1x%dx128x1024" % S
            hbm(nm, lambda: K.lib.softmax_q19(R.data_ptr(), Cs.data_ptr(), K.EXP2_FRAC_LUT_Q19.data_ptr(), 1, S, 128, 1024),
                R.numel(), steps=10, sample=softmax_sample(nm, R, Cs, "softmax_q19"))
            if S == 1024:       # the Q21 variant (no live caller in the reference's model) on the same rows
                K.softmax_init_q21()
                nm = "softmax_q21_1x1024x128x1024"
                hbm(nm, lambda: K.lib.softmax_q21(R.data_ptr(), Cs.data_ptr(), K.EXP2_FRAC_LUT_Q21.data_ptr(), 1, S, 128, 1024),
                    R.numel(), steps=10, sample=softmax_sample(nm, R, Cs, "softmax_q21"))
            del R, Cs
        for S in (512, 8192):
            g2 = torch.Generator(device="cpu").manual_seed(2300 + S)
            R = randint(g2, -(16 << 23), 16 << 23, (1, S, 18432)).cuda()
            Cs = torch.empty_like(R)
            for nm, fn in (("silu_q23", K.lib.silu_q23), ("sigmoid_q23", K.lib.sigmoid_q23)):
                hbm("%s_1x%dx18432" % (nm, S),
                    lambda fn=fn: fn(R.data_ptr(), Cs.data_ptr(), K.EXP2_FRAC_LUT_Q23.data_ptr(), 1, S, 18432),
                    R.numel(), steps=20, sample=act_sample("%s_1x%dx18432" % (nm, S), R, Cs, nm))
            if S == 8192:       # the Q25 variants (bound at import only in the reference)
                K.silu_init_q25()
                for nm, fn in (("silu_q25", K.lib.silu_q25), ("sigmoid_q25", K.lib.sigmoid_q25)):
                    hbm("%s_1x%dx18432" % (nm, S),
                        lambda fn=fn: fn(R.data_ptr(), Cs.data_ptr(), K.EXP2_FRAC_LUT_Q25.data_ptr(), 1, S, 18432),
                        R.numel(), steps=20, sample=act_sample("%s_1x%dx18432" % (nm, S), R, Cs, nm))
            del R, Cs
        g6 = torch.Generator(device="cpu").manual_seed(600)
        for Mr in (500, 16384):
            Ar = randint(g6, -(1 << 37), 1 << 37, (Mr, 7168)).cuda()
            Wr = randint(g6, 1 << 18, 1 << 20, (7168,)).to(torch.int32).cuda()
            rr = torch.empty((Mr,), dtype=torch.int64, device="cuda")
            Cr = torch.empty_like(Ar)
            hbm("rmsnorm_fused_%dx7168" % Mr,
                lambda: K.lib.rms_norm_fused_32(Ar.data_ptr(), Wr.data_ptr(), rr.data_ptr(), Cr.data_ptr(), Mr, 7168, 1, 7168),
                Ar.numel(), extra_bytes=4.0 * 7168 + 8.0 * Mr, steps=20, sample=rms_sample("rmsnorm_fused_%dx7168" % Mr, Ar, Wr, rr, Cr))
            if Mr == 16384:
                # the residual connection in front of the norm, fused (32 B/element) against torch's multiply and add
                # followed by the fused norm (model.py:1465-1468)
                Yr = randint(g6, -(1 << 25), 1 << 25, (Mr, 7168)).cuda()
                Xo = torch.empty_like(Ar)
                nm = "rmsnorm_residual_fused_%dx7168_32B_per_element" % Mr
                hbm(nm, lambda: K.lib.rms_norm_residual_fused_32(Ar.data_ptr(), Yr.data_ptr(), 12, Wr.data_ptr(), Xo.data_ptr(),
                                                                 rr.data_ptr(), Cr.data_ptr(), Mr, 7168, 1, 7168),
                    Ar.numel(), bytes_per_elem=32.0, steps=20)

                def chain0():
                    xn = Ar + Yr * (1 << 12)
                    K.lib.rms_norm_fused_32(xn.data_ptr(), Wr.data_ptr(), rr.data_ptr(), Cr.data_ptr(), Mr, 7168, 1, 7168)

                extra[nm]["unfused_chain_ms"] = timed(K, chain0, 5, 2)
                del Yr, Xo
            del Ar, Cr

        # the two fusions against the chains they replace (the reference's tensor ops around the kernel, on torch)
        g7 = torch.Generator(device="cpu").manual_seed(3300)
        s1 = randint(g7, -(6 << 20), 6 << 20, (1, 1024, 128, 1024)).cuda()
        s2 = randint(g7, -(6 << 20), 6 << 20, (1, 1024, 128, 1024)).cuda()
        msk = torch.full((1024, 1024), -(64 << 36), dtype=torch.int64).triu_(1).cuda()
        sc = torch.empty_like(s1)
        pr = torch.empty_like(s1)
        hbm("softmax_q19_scores_fused_1x1024x128x1024_32B_per_element",
            lambda: K.softmax_q19_scores(s1, s2, msk, pr, sc), s1.numel(), bytes_per_elem=32.0, steps=10)

        def chain():
            x = (s1 + s2) * 94 // 695
            x += msk.unsqueeze(1)
            K.lib.softmax_q19(x.data_ptr(), pr.data_ptr(), K.EXP2_FRAC_LUT_Q19.data_ptr(), 1, 1024, 128, 1024)

        ms_chain = timed(K, chain, 5, 2)
        extra["softmax_q19_scores_fused_1x1024x128x1024_32B_per_element"]["unfused_chain_ms"] = ms_chain
        del s1, s2, sc, pr
        g8 = torch.Generator(device="cpu").manual_seed(2400)
        r1 = randint(g8, -(16 << 23), 16 << 23, (1, 8192, 18432)).cuda()
        r2 = randint(g8, -(16 << 23), 16 << 23, (1, 8192, 18432)).cuda()
        hh = torch.empty_like(r1)
        hbm("silu_mul_q23_fused_1x8192x18432_24B_per_element", lambda: K.silu_mul_q23(r1, r2, hh), r1.numel(),
            bytes_per_elem=24.0, steps=10)

        def chain2():
            K.lib.silu_q23(r1.data_ptr(), hh.data_ptr(), K.EXP2_FRAC_LUT_Q23.data_ptr(), 1, 8192, 18432)
            torch.bitwise_right_shift(hh * r2, 23, out=hh)

        extra["silu_mul_q23_fused_1x8192x18432_24B_per_element"]["unfused_chain_ms"] = timed(K, chain2, 5, 2)
        del r1, r2, hh

        # expert routing of the gate: 256 experts in 8 groups, 4 groups kept, top 8 (8*256 + 2*8*8 bytes per token)
        gr = torch.Generator(device="cpu").manual_seed(800)
        gbias = randint(gr, -(1 << 18), 1 << 18, (256,)).to(torch.int32).cuda()
        for Tt in (256, 65536):
            gsc = randint(gr, 1, 1 << 23, (Tt, 256)).cuda()
            hbm("gate_route_%dx256" % Tt, lambda: K.gate_route(gsc, gbias, 8, 4, 8), Tt, bytes_per_elem=8.0 * 256 + 128.0, steps=20)
            # sigmoid and routing in one launch, from the gate's logits (the scores not written: the same bytes)
            glog = randint(gr, -(1 << 25), 1 << 25, (Tt, 256)).cuda()
            hbm("gate_sigmoid_route_%dx256" % Tt, lambda: K.gate_sigmoid_route(glog, gbias, 8, 4, 8, keep_scores=False), Tt,
                bytes_per_elem=8.0 * 256 + 128.0, steps=20)
            gsig = torch.empty_like(glog)

            def two_launches():
                K.sigmoid_q23(glog[None], gsig[None])
                K.gate_route(gsig, gbias, 8, 4, 8)

            extra["gate_sigmoid_route_%dx256" % Tt]["unfused_chain_ms"] = timed(K, two_launches, 20, 3)
            del gsc, glog, gsig

        # config 5's routed experts: 256 tokens, top 8 of 256 experts of width 2048 on dim 7168, int64 weights resident
        # (90.2 GB): bound by the one pass over the weights.  Routing, dispatch, three grouped GEMM launches, combine.
        free_b, _tot = torch.cuda.mem_get_info()
        if free_b > 110 * (1 << 30):
            gm = torch.Generator(device="cuda").manual_seed(5001)
            mkw = lambda *shape: torch.randint(-(1 << 16), 1 << 16, shape, generator=gm, dtype=torch.int64, device="cuda")
            ew1 = [mkw(2048, 7168) for _ in range(256)]
            ew3 = [mkw(2048, 7168) for _ in range(256)]
            ew2 = [mkw(7168, 2048) for _ in range(256)]
            tabs = [K.pointer_table(w) for w in (ew1, ew3, ew2)]
            xm = randint(gr, -(1 << 20), 1 << 20, (256, 7168)).cuda()
            sm = randint(gr, 1, 1 << 23, (256, 256)).cuda()
            wm, im = K.gate_route(sm, gbias, 8, 4, 8)
            wbytes = 3.0 * 256 * 2048 * 7168 * 8
            hbm("moe_experts_config5_256tok_top8_of_256", lambda: K.moe_experts(xm, wm, im, tabs[0], tabs[1], tabs[2], False, 2048, 17, 20),
                1, bytes_per_elem=wbytes, steps=3)
            extra["moe_experts_config5_256tok_top8_of_256"]["weight_bytes"] = wbytes
            # the same with the experts' weights prepared once as digit planes (3 bytes per weight instead of 8)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for tb in tabs:
                K.prepare_weights(tb, groups=256, N=int(2048 if tb is not tabs[2] else 7168), K=int(7168 if tb is not tabs[2] else 2048))
            prep_ms = (time.perf_counter() - t0) * 1e3
            hbm("moe_experts_config5_prepared_weights", lambda: K.moe_experts(xm, wm, im, tabs[0], tabs[1], tabs[2], False, 2048, 17, 20),
                1, bytes_per_elem=wbytes * 3.0 / 8.0, steps=3)
            extra["moe_experts_config5_prepared_weights"]["plane_bytes"] = wbytes * 3.0 / 8.0
            extra["moe_experts_config5_prepared_weights"]["prepare_once_ms"] = prep_ms
            for tb in tabs:
                K.release_weights(tb)
            del ew1, ew3, ew2, tabs
            torch.cuda.empty_cache()
            # the same with the model's weight type: int32 at 31 bits (45 GB), shifts that keep the activations in Q23
            # range; 256 tokens (three grouped MFMA launches) and one token (three grouped matrix-vector launches)
            mk32 = lambda *shape: torch.randint(-(1 << 30), 1 << 30, shape, generator=gm, dtype=torch.int64, device="cuda").to(torch.int32)
            ew1 = [mk32(2048, 7168) for _ in range(256)]
            ew3 = [mk32(2048, 7168) for _ in range(256)]
            ew2 = [mk32(7168, 2048) for _ in range(256)]
            tabs = [K.pointer_table(w) for w in (ew1, ew3, ew2)]
            for Tt in (256, 1):
                wt, it = wm[:Tt].contiguous(), im[:Tt].contiguous()
                xt = xm[:Tt].contiguous()
                hit = int(torch.unique(it).numel())
                wbytes = 3.0 * hit * 2048 * 7168 * 4
                nm = "moe_experts_int32_%dtok_top8_of_256" % Tt
                hbm(nm, lambda: K.moe_experts(xt, wt, it, tabs[0], tabs[1], tabs[2], True, 2048, 30, 33), 1, bytes_per_elem=wbytes, steps=3)
                extra[nm]["weight_bytes"] = wbytes
                extra[nm]["experts_hit"] = hit
                if Tt == 256:
                    # The same with activation buffers the library has not seen: the legs above hand it the same
                    # addresses call after call (torch's allocator returns them), so its remembered digit counts hit.
                    # Here every call's intermediates land on new memory (a growing pile of blocks keeps the old
                    # addresses taken): what a layer pays whose buffers move.  Wall clock, since such a call waits.
                    pile = []

                    def fresh_call():
                        pile.append(torch.empty((Tt * 8 * 7168 + 4096 * len(pile),), dtype=torch.int64, device="cuda"))
                        return K.moe_experts(xt, wt, it, tabs[0], tabs[1], tabs[2], True, 2048, 30, 33)

                    fresh_call()
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    for _ in range(3):
                        fresh_call()
                    torch.cuda.synchronize()
                    extra[nm]["ms_with_activation_buffers_at_new_addresses"] = (time.perf_counter() - t0) * 1e3 / 3
                    del pile
            # 256 tokens again with the int32 weights prepared as digit planes (four bytes per weight, as before, but
            # nothing of B is split in the kernel)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for tb in tabs:
                K.prepare_weights(tb, groups=256, N=int(2048 if tb is not tabs[2] else 7168), K=int(7168 if tb is not tabs[2] else 2048), b32=True)
            prep_ms = (time.perf_counter() - t0) * 1e3
            hit = int(torch.unique(im).numel())
            wbytes = 3.0 * hit * 2048 * 7168 * 4
            nm = "moe_experts_int32_256tok_prepared_weights"
            hbm(nm, lambda: K.moe_experts(xm, wm, im, tabs[0], tabs[1], tabs[2], True, 2048, 30, 33), 1, bytes_per_elem=wbytes, steps=3)
            extra[nm]["weight_bytes"] = wbytes
            extra[nm]["prepare_once_ms"] = prep_ms
            for tb in tabs:
                K.release_weights(tb)
            del ew1, ew3, ew2, tabs
            torch.cuda.empty_cache()

        # witness dump: what one layer's ~30 saveTensor calls cost the host thread, against the reference's way
        # (synchronous .cpu() + tobytes + write, inference/model.py:94-102); files go to a temporary directory
        import shutil
        import tempfile
        tmpd = tempfile.mkdtemp(prefix="zkdump_")
        try:
            dumps = [randint(gr, -(1 << 40), 1 << 40, (256, 7168)).cuda() for _ in range(30)]
            torch.cuda.synchronize()

            def ref_style():
                for i, t in enumerate(dumps):
                    with open(os.path.join(tmpd, "r%d.bin" % i), "wb") as f:
                        f.write(t.cpu().contiguous().numpy().tobytes(order="C"))

            ref_style()
            t0 = time.perf_counter()
            ref_style()
            ref_ms = (time.perf_counter() - t0) * 1e3
            for rep in range(2):
                t0 = time.perf_counter()
                for i, t in enumerate(dumps):
                    K.saveTensor(os.path.join(tmpd, "a%d.bin" % i), t)
                queued_ms = (time.perf_counter() - t0) * 1e3
                K.dump_flush()
                total_ms = (time.perf_counter() - t0) * 1e3
            nbytes = sum(t.numel() * 8 for t in dumps)
            extra["witness_dump_30x256x7168"] = {"bytes": nbytes, "host_blocked_ms": queued_ms, "until_flushed_ms": total_ms,
                                                 "reference_style_ms": ref_ms}
            del dumps
        finally:
            shutil.rmtree(tmpd, ignore_errors=True)

        # one token (a decoding step, and the head on every pass): weight streams, reported by the bytes of W per second
        gd = torch.Generator(device="cuda").manual_seed(1100)

        def gemv_leg(name, Kd, N, w32, b_rs, bits_w):
            Ad = torch.randint(-(1 << 37), 1 << 37, (1, 1, Kd), generator=gd, dtype=torch.int64, device="cuda")
            Wd = torch.randint(-(1 << bits_w), 1 << bits_w, (N, Kd), generator=gd, dtype=torch.int64, device="cuda")
            if w32:
                Wd = Wd.to(torch.int32)
            Cd = torch.empty((1, 1, N), dtype=torch.int64, device="cuda")
            fn = K.lib.int64_32_bmm_broadcast_launcher if w32 else K.lib.int64_64_bmm_broadcast_launcher
            call = lambda: fn(Ad.data_ptr(), Wd.data_ptr(), Cd.data_ptr(), None, 1, b_rs, 29, 1, 1, Kd, N)
            hbm(name, call, N * Kd, bytes_per_elem=4.0 if w32 else 8.0, steps=20)
            samples.append(gemm_sample(name, Ad, Wd, Cd, None, 29, b_rs=b_rs, rows=1, cols=128))
            extra[name]["path"] = {1: "valu", 2: "mfma_i8"}.get(K.gemm_last_plan()[0], "?")

        gemv_leg("gemm_1token_head_7168x129280_int64_div256", 7168, 129280, False, 256, 43)
        gemv_leg("gemm_1token_wo_16384x7168_int32", 16384, 7168, True, 1, 31)
        gemv_leg("gemm_1token_wkv_a_7168x576_int32", 7168, 576, True, 1, 31)

        # the four MLA einsums at config 3's shape (S = T = 1024, 128 heads, absorb mode: model.py:884-936), Q30
        # activations against Q24 cache entries / int32 Q25 weights
        ge = torch.Generator(device="cuda").manual_seed(900)
        rnd = lambda bits, *shape: torch.randint(-(1 << bits), 1 << bits, shape, generator=ge, dtype=torch.int64, device="cuda")

        def einsum_leg(name, fn, macs, which=None, a=None, b=None, rescale=0):
            out = fn()
            K._check(name)
            if which is not None:
                # two sequence positions of A against the whole of B, kept for the CPU leg's 128-bit check
                si = sample_rows(a.shape[1], 2, 19)
                ah, bh = a[:, si].cpu().numpy(), b.cpu().numpy()
                oh = out[:, si].cpu().numpy()

                def check(ck, np, which=which, ah=ah, bh=bh, oh=oh, rescale=rescale):
                    if not np.array_equal(getattr(ck, which)(np.ascontiguousarray(ah), bh, rescale), oh):
                        raise Mismatch("%s: sampled positions differ from the CPU restatement" % name)
                    return "%d sampled sequence positions equal the 128-bit CPU restatement" % len(si)
                samples.append((name, check))
            del out
            ms = timed(K, fn, 5, 2)
            K._check(name)
            _p, la, lb = K.gemm_last_plan()
            extra[name] = {"ms": ms, "gmacs": macs / ms / 1e6, "macs": macs, "limbs_a": la, "limbs_b": lb,
                           "digit_pairs": K.gemm_last_pairs()}

        Se, He, Ce, De, Re = 1024, 128, 512, 128, 64
        qn, wb1 = rnd(30, 1, Se, He, De), rnd(25, He, De, Ce).to(torch.int32)
        einsum_leg("einsum_bshd_hdc_bshc_1x1024x128x128_to_512", lambda: K.einsum_bshd_hdc_bshc(qn, wb1, 21), Se * He * De * Ce,
                   "einsum_bshd_hdc_bshc", qn, wb1, 21)
        del qn, wb1
        qa, kvc = rnd(30, 1, Se, He, Ce), rnd(24, 1, Se, Ce)
        einsum_leg("einsum_bshc_btc_bsht_1x1024x128x512_T1024", lambda: K.einsum_bshc_btc_bsht(qa, kvc, 23), Se * He * Se * Ce,
                   "einsum_bshc_btc_bsht", qa, kvc, 23)
        del qa
        qp, pec = rnd(30, 1, Se, He, Re), rnd(24, 1, Se, Re)
        einsum_leg("einsum_bshc_btc_bsht_1x1024x128x64_T1024", lambda: K.einsum_bshc_btc_bsht(qp, pec, 21), Se * He * Se * Re,
                   "einsum_bshc_btc_bsht", qp, pec, 21)
        del qp, pec
        pp = torch.randint(0, 1 << 19, (1, Se, He, Se), generator=ge, dtype=torch.int64, device="cuda")
        einsum_leg("einsum_bsht_btc_bshc_1x1024x128xT1024_to_512", lambda: K.einsum_bsht_btc_bshc(pp, kvc, 23), Se * He * Se * Ce,
                   "einsum_bsht_btc_bshc", pp, kvc, 23)
        del pp, kvc
        # config 3 as the benchmark set states it: Q [1,1024,128,192] against K [1,1024,192] in one call, P.V with 128 columns
        q3, k3 = rnd(16, 1, Se, He, 192), rnd(16, 1, Se, 192)
        einsum_leg("einsum_bshc_btc_bsht_config3_1x1024x128x192_T1024", lambda: K.einsum_bshc_btc_bsht(q3, k3, 21), Se * He * Se * 192,
                   "einsum_bshc_btc_bsht", q3, k3, 21)
        config3_host = {"q": q3[:, :16].cpu(), "k": k3.cpu(), "scores": K.einsum_bshc_btc_bsht(q3, k3, 21)[:, :16].cpu()}
        del q3, k3
        p3 = torch.randint(0, 1 << 19, (1, Se, He, Se), generator=ge, dtype=torch.int64, device="cuda")
        v3 = rnd(16, 1, Se, 128)
        einsum_leg("einsum_bsht_btc_bshc_config3_1x1024x128xT1024_to_128", lambda: K.einsum_bsht_btc_bshc(p3, v3, 23), Se * He * Se * 128,
                   "einsum_bsht_btc_bshc", p3, v3, 23)
        config3_host.update({"p": p3[:, :16].cpu(), "v": v3.cpu(), "out": K.einsum_bsht_btc_bshc(p3, v3, 23)[:, :16].cpu()})
        del p3, v3
        oo, wb2 = rnd(30, 1, Se, He, Ce), rnd(25, He, De, Ce).to(torch.int32)
        einsum_leg("einsum_bshc_hdc_bshd_1x1024x128x512_to_128", lambda: K.einsum_bshc_hdc_bshd(oo, wb2, 21), Se * He * De * Ce,
                   "einsum_bshc_hdc_bshd", oo, wb2, 21)
        del oo, wb2

        # RoPE and the float -> fixed converters (weight-loading path), by their own algorithmic bytes per element
        gq = torch.Generator(device="cpu").manual_seed(700)
        q_pe = randint(gq, -(1 << 30), 1 << 30, (1, 4096, 128, 32, 2)).cuda()
        tab = randint(gq, -(1 << 42), 1 << 42, (1, 4096, 1, 32, 2)).cuda()
        out = torch.empty_like(q_pe)
        hbm("rope_1x4096x128x64", lambda: K.lib.complex_int64_mul(q_pe.data_ptr(), tab.data_ptr(), out.data_ptr(), 1, 4096, 128, 32),
            q_pe.numel(), steps=20)
        del q_pe, out
        # checkpoint quantisation (convert2.py): block-scaled fp8 weights -> int32, 1 byte read + 4 written per weight
        w8 = torch.randint(0, 256, (18432, 7168), generator=gq, dtype=torch.uint8).cuda()
        s8 = (torch.rand((144, 56), generator=gq, dtype=torch.float32) * 1e-3 + 1e-5).cuda()
        o8 = torch.empty((18432, 7168), dtype=torch.int32, device="cuda")
        hbm("fp8_block_scaled_to_int32_18432x7168", lambda: K.lib.fp8_block_scaled_to_int32(w8.data_ptr(), s8.data_ptr(), o8.data_ptr(), 18432, 7168, 30),
            w8.numel(), bytes_per_elem=5.0, steps=20)
        # four fifths of that kernel's traffic are writes: next to it, what this device takes in streaming stores alone
        store_gbps = K.lib.zk_probe_store_gbps(528 << 20, 10)
        K._check("store probe")
        e8 = extra["fp8_block_scaled_to_int32_18432x7168"]
        e8["streaming_store_ceiling_GBps"] = store_gbps
        e8["write_GBps"] = 4.0 * w8.numel() / (e8["ms"] * 1e-3) / 1e9
        e8["write_frac_of_store_ceiling"] = e8["write_GBps"] / store_gbps if store_gbps else None
        del w8, o8
        wb = torch.randn((18432, 7168), generator=gq, dtype=torch.float32)
        w16 = wb.to(torch.bfloat16).cuda()
        o32 = torch.empty((18432, 7168), dtype=torch.int32, device="cuda")
        hbm("bf16_to_int32_18432x7168", lambda: K.lib.bf16_to_int32_2d(w16.data_ptr(), o32.data_ptr(), 18432, 7168, 20),
            w16.numel(), bytes_per_elem=6.0, steps=20)
        w32 = wb.cuda()
        o64 = torch.empty((18432, 7168), dtype=torch.int64, device="cuda")
        hbm("float32_to_int64_18432x7168", lambda: K.lib.float32_to_int64_2d(w32.data_ptr(), o64.data_ptr(), 18432, 7168, 5),
            w32.numel(), bytes_per_elem=12.0, steps=20)
        del wb, w16, o32, w32, o64

    if "calib" in legs:
        # plain copy of known size (1 GiB in, 1 GiB out): what FETCH_SIZE / WRITE_SIZE read for it is the
        # scale factor applied to the same counters of the GEMM kernel (see profiles/)
        src = torch.empty((1 << 27,), dtype=torch.int64, device="cuda").fill_(3)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---------------- checks and the CPU baseline, before anything is reported ----------------
    cpu_baseline = None
    if "cpu" in legs:
        cpu_baseline = cpu_leg(A_h, W_h, c, Cb, Rb, samples, verified,
                               locals().get("full_range_host"), locals().get("config3_host"))
    else:
        verified["other_legs"] = "not compared in this run (--no-cpu skips the CPU leg that holds the comparisons)"

    # Rooflines of the other shapes the metric names, from this run's HIP-event timings.  They live INSIDE "roofline" as
    # flat numbers (the record a driver keeps of this line may hold known keys only and drop nested objects), and once
    # more, with their notes, under roofline["others"].
    others = {}
    flat = {}
    if "gemm_config1_16x7168x576" in extra:
        e = extra["gemm_config1_16x7168x576"]
        wbytes = 8.0 * (576 * 7168 + 16 * 7168 + 2 * 16 * 576)
        gbs = wbytes / (e["ms"] * 1e-3) / 1e9
        others["gemm_config1_16x7168x576"] = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                                              "traffic": measured_traffic("gemm_config1_bytes_per_call"),
                                              "traffic_source": "committed rocprofv3 --pmc profile of this call (profiles/gemm_config1_rows16_hbm_traffic.md), "
                                                                "NOT measured in this run",
                                              "note": "algorithmic bytes 8*(N*K + M*K + 2*M*N) = %.0f per call: the weights are streamed once" % wbytes}
        flat["gemm_config1_us"] = e["ms"] * 1e3
        flat["gemm_config1_gmacs"] = e["gmacs"]
        flat["gemm_config1_GBps"] = gbs
        flat["gemm_config1_frac_hbm"] = gbs / HBM_PEAK_GBS
        flat["gemm_config1_traffic"] = measured_traffic("gemm_config1_bytes_per_call")
        if launch_floor_us is not None:
            # what two dependent launches cost on this device whatever they compute, plus the weights at the HBM peak
            floor_us = launch_floor_us + wbytes / (HBM_PEAK_GBS * 1e9) * 1e6
            flat["gemm_config1_two_launch_floor_us"] = launch_floor_us
            flat["gemm_config1_frac_of_launch_floor_plus_hbm"] = floor_us / (e["ms"] * 1e3)
    for nm, short in (("gemm_config2_w1_128x7168x2048", "gemm_config2_w1_us"), ("gemm_config2_w2_128x2048x7168", "gemm_config2_w2_us")):
        if nm in extra:
            flat[short] = extra[nm]["ms"] * 1e3
    if "gemm_config4_prepared_weights" in extra:
        # the headline product on weights prepared once (not `value`): its time and the same i8 operation count over it
        e = extra["gemm_config4_prepared_weights"]
        flat["gemm_config4_prepared_us"] = e["ms"] * 1e3
        flat["gemm_config4_prepared_frac_mfma_peak"] = 2.0 * e["digit_pairs"] * e["macs"] / (e["ms"] * 1e-3) / 1e12 / I8_MFMA_PEAK_TOPS
    for nm in ("softmax_q19_1x1024x128x1024", "softmax_q19_1x4096x128x1024", "silu_q23_1x512x18432", "silu_q23_1x8192x18432",
               "sigmoid_q23_1x512x18432", "sigmoid_q23_1x8192x18432", "rmsnorm_fused_500x7168", "rmsnorm_fused_16384x7168"):
        if nm in extra:
            e = extra[nm]
            others[nm] = {"bound": "hbm", "achieved": e["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": e["frac_hbm_peak"],
                          "traffic": None, "note": "16 algorithmic bytes per element (8 read + 8 written)"}
            flat[nm + "_GBps"] = e["GBps"]
            flat[nm + "_frac_hbm"] = e["frac_hbm_peak"]
            if "frac_of_launch_plus_hbm_floor" in e:
                flat[nm + "_frac_of_launch_plus_hbm_floor"] = e["frac_of_launch_plus_hbm_floor"]
    for nm in ("gemm_1token_wkv_a_7168x576_int32",):
        if nm in extra and "frac_of_launch_plus_hbm_floor" in extra[nm]:
            flat[nm + "_us"] = extra[nm]["ms"] * 1e3
            flat[nm + "_frac_of_launch_plus_hbm_floor"] = extra[nm]["frac_of_launch_plus_hbm_floor"]
    for nm in ("moe_experts_int32_256tok_top8_of_256", "moe_experts_config5_256tok_top8_of_256"):
        if nm in extra:
            flat[nm + "_frac_hbm"] = extra[nm]["frac_hbm_peak"]
    if "moe_experts_int32_256tok_top8_of_256" in extra:
        # (counter traffic of the layer's three grouped launches against their algorithmic bytes, from the committed profile)
        flat["moe_experts_int32_gemm_traffic"] = measured_traffic("moe_experts_int32_gemm_bytes_per_call")
        flat["moe_experts_int32_gemm_algorithmic_bytes"] = measured_traffic("moe_experts_int32_gemm_algorithmic_bytes_per_call")
    roofline.update(flat)
    roofline["others"] = others
    cold = {}
    for nm, short in (("cold_gemm_config4_512x7168x18432", "config4"), ("cold_gemm_config2_w1_128x7168x2048", "config2_w1"),
                      ("cold_gemm_config1_16x7168x576", "config1")):
        if nm in extra:
            e = extra[nm]
            cold[short + "_first_call_ms"] = e["first_call_new_addresses_ms"]
            cold[short + "_warm_call_ms"] = e["warm_single_call_ms"]
            cold[short + "_recycled_wider_ms"] = e["recycled_address_wider_contents_ms"]
    all_checked = "cpu" in legs

    config = {"workload": "config4: int64 GEMM Y[512,18432] = X[512,7168] @ W[18432,7168]^T, int64 W, "
                          "X in [-2^20,2^20), W in [-2^16,2^16), c_rescale=29, C and R written",
              "path": {1: "valu", 2: "mfma_i8"}.get(path, "?"), "limbs_a": la, "limbs_b": lb,
              "kernel_ms_hip_events": kern_ms,
              "verified": bool(all_checked),
              "untimed_calls_before_the_timed_steps": untimed_calls,
              "untimed_calls_note": "warmup steps asked for plus calls keeping the device busy %d ms (idle clocks)" % SPIN_UP_MS}
    if "gemm_config1_us" in flat:
        config["gemm_config1_us"] = flat["gemm_config1_us"]
    config.update(cold)
    # the figures a reader wants first, once more at the very end of the line (a record that keeps only the tail of the
    # output still holds them)
    summary = {"value_gmacs": value, "ms_per_step": ms_per_step, "roofline_frac": roofline.get("frac"), "verified": bool(all_checked)}
    summary.update({k: v for k, v in flat.items() if k.endswith(("_us", "_frac_hbm", "_frac_mfma_peak"))})
    summary.update(cold)
    if cpu_baseline:
        summary["cpu_baseline_gmacs"] = cpu_baseline.get("value")
    out = {
        "metric": "int64 GEMM Gmac/s @7168x576 & 18432x7168 + softmax/SiLU HBM GB/s, 1 MI355X",
        "value": value, "unit": "Gmac/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int64", "data": "synthetic",
        "config": config,
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
        "verified": verified,
        "extra": extra,
        "summary": summary,
    }
    # everything is released and flushed before the line is printed, so that nothing lingers behind it
    K.dump_flush()
    del A, W, Cb, Rb
    torch.cuda.empty_cache()
    torch.cuda.synchronize()
    # this program starts no other process (no subprocess, no worker pool; the CPU leg's threads live in this process and
    # end with it): whatever a supervisor finds alive once it has exited is not its child.  Said in the line, checked here.
    try:
        import psutil
        out["summary"]["child_processes_at_exit"] = len(psutil.Process().children(recursive=True))
    except Exception:
        out["summary"]["child_processes_at_exit"] = None
    print(json.dumps(out))
    sys.stdout.flush()
    sys.stderr.flush()
    # Nothing is left to do: leave without the interpreter's teardown of a process that held 90 GB of tensors.  A
    # profiler that wraps the run (rocprofv3 exports ROCPROF* variables to it) writes its files when the process ends
    # the ordinary way, so under one the ordinary way it is.
    if not any(k.startswith("ROCPROF") for k in os.environ):
        os._exit(0)


def measured_traffic(key="gemm_config4_bytes_per_launch"):
    """HBM bytes per launch of the config-4 GEMM kernel (or, with another key, per call of config 1), from the committed
    rocprofv3 --pmc runs (FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter reads for a 1 GiB copy):
    profiles/traffic.json."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f).get(key)
    except (OSError, ValueError):
        return None


def cpu_leg(A_h, W_h, c, Cb, Rb, samples, verified, full_range_host, config3_host):
    """The reference's CPU path for a Linear layer is torch's int64 matmul on CPU tensors followed by the shift
    (the generic branch of `linear`, inference/model.py:179-181).  Timed on a column block of config 4 sized to take
    roughly 10 s with all host cores, then with the reference's own 8 threads (inference/generate.py:333) and with one;
    the GPU's result for the same columns is compared with it bit for bit.  Config 1, the full-range variant at shift 0
    and config 3's two attention einsums (inference/model.py:884-936) run on the same CPU path.  The fixed-point kernels
    have no CPU form in the reference: this build's scalar C restatement is timed instead (labelled as such), and the
    same restatement checks the samples the GPU legs kept."""
    import torch
    cores = os.cpu_count() or 1
    try:
        cores = min(cores, len(os.sched_getaffinity(0)))
    except AttributeError:
        pass
    omp = int(os.environ.get("OMP_NUM_THREADS", "0") or 0)
    if omp > 0:
        cores = min(cores, omp)
    A2 = A_h[0]
    M, Kd = A2.shape

    def run(lo, ncols, threads):
        torch.set_num_threads(threads)
        Wt = W_h[lo:lo + ncols].T.contiguous()
        t0 = time.perf_counter()
        prod = torch.matmul(A2, Wt)
        y = prod >> c
        dt = time.perf_counter() - t0
        return dt, prod, y

    dt, _, _ = run(0, 16, cores)                                  # calibrate
    rate = M * Kd * 16 / dt
    ncols = int(min(W_h.shape[0], max(64, (rate * 10.0) // (M * Kd))))
    dt, prod, y = run(0, ncols, cores)
    # the GPU's columns against the product just computed: quotient and rebuilt product
    Cg, Rg = Cb[0, :, :ncols].cpu(), Rb[0, :, :ncols].cpu()
    if not torch.equal(Cg, y) or not torch.equal((Cg << c) + Rg, prod):
        raise Mismatch("config-4 GEMM: the GPU result differs from torch's CPU int64 matmul on columns [0, %d)" % ncols)
    verified["gemm_config4_cpu_block"] = "C and C*2^c+R equal the timed CPU product on columns [0, %d)" % ncols
    macs = M * Kd * ncols
    res = {"value": macs / dt / 1e9, "unit": "Gmac/s", "cores": cores, "kind": "reference",
           "sample": "torch.matmul int64 on CPU then >> %d (the reference's F.linear CPU branch, model.py:179-181) on "
                     "X[512,7168] x W[:%d,7168]^T of config 4, %.1f s" % (c, ncols, dt)}
    del prod, y, Cg, Rg
    n8 = max(64, ncols // 2)
    dt8, _, _ = run(0, n8, min(8, cores))
    res["value_8_threads"] = M * Kd * n8 / dt8 / 1e9
    n1 = max(16, ncols // (2 * cores))
    dt1, _, _ = run(0, n1, 1)
    res["value_1_thread"] = M * Kd * n1 / dt1 / 1e9

    # config 1 on the same CPU path (Y[16,576] = X[16,7168] @ W[576,7168]^T), all cores and 8 threads
    g1 = torch.Generator(device="cpu").manual_seed(1000)
    X1 = randint(g1, -(1 << 20), 1 << 20, (16, 7168))
    W1t = randint(g1, -(1 << 16), 1 << 16, (576, 7168)).T.contiguous()
    for key, threads in (("config1_gmacs", cores), ("config1_gmacs_8_threads", min(8, cores))):
        torch.set_num_threads(threads)
        torch.matmul(X1, W1t)
        ts = []
        for _ in range(7):
            t0 = time.perf_counter()
            _y1 = torch.matmul(X1, W1t) >> c
            ts.append(time.perf_counter() - t0)
        res[key] = 16 * 7168 * 576 / sorted(ts)[len(ts) // 2] / 1e9
    torch.set_num_threads(cores)

    # config 4 with full-range operands at shift 0 (the product modulo 2^64): a block of 256 columns
    if full_range_host is not None:
        Af_h, Wf_h = full_range_host
        Wt = Wf_h.T.contiguous()
        t0 = time.perf_counter()
        _yf = torch.matmul(Af_h[0], Wt)
        dtf = time.perf_counter() - t0
        res["config4_full_range_shift0_gmacs"] = Af_h.shape[1] * Af_h.shape[2] * Wf_h.shape[0] / dtf / 1e9

    # config 3: scores = (Q K^T + 10) >> 21 and P V with (sum + 11) >> 23 on 16 of the 1024 sequence positions (the
    # rounding term of the reference's kernels is half the shift COUNT, inference/int64_gemm.cu:442); the GPU's rows
    # for the same positions are compared
    if config3_host is not None:
        h = config3_host
        t0 = time.perf_counter()
        sc = (torch.einsum("bshc,btc->bsht", h["q"], h["k"]) + 10) >> 21
        dts = time.perf_counter() - t0
        t0 = time.perf_counter()
        pv = (torch.einsum("bsht,btc->bshc", h["p"], h["v"]) + 11) >> 23
        dtp = time.perf_counter() - t0
        if not torch.equal(sc, h["scores"]) or not torch.equal(pv, h["out"]):
            raise Mismatch("config 3: the GPU einsums differ from torch.einsum on the CPU")
        verified["config3_einsums"] = "scores and P.V equal torch.einsum int64 on the CPU on 16 of 1024 sequence positions"
        res["config3_qk_gmacs"] = h["q"].shape[1] * 128 * 1024 * 192 / dts / 1e9
        res["config3_pv_gmacs"] = h["p"].shape[1] * 128 * 1024 * 128 / dtp / 1e9

    # The reference has no CPU implementation of its fixed-point kernels; what is timed here is this build's scalar
    # C restatement of them (OpenMP over rows), labelled as such: "oracle, not reference".  The same restatement is the
    # checker for the samples the GPU legs kept.
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import numpy as np
    import oracle
    oracle.set_threads(cores)
    for name, check in samples:
        verified[name] = check(oracle, np)
    try:
        rng = np.random.default_rng(7)
        others = {}

        def leg(name, fn, nelem, what):
            entry = {"unit": "GB/s at 16 B/element", "kind": "port (oracle, not reference)"}
            for threads, key, budget in ((cores, "value", 1.5), (1, "value_1_thread", 1.0)):
                oracle.set_threads(threads)
                fn()
                reps, t0 = 0, time.perf_counter()
                while reps < 2 or time.perf_counter() - t0 < budget:
                    fn()
                    reps += 1
                dt = (time.perf_counter() - t0) / reps
                entry[key] = nelem * 16.0 / dt / 1e9
            entry["cores"] = cores
            entry["sample"] = what
            others[name] = entry

        xs = rng.integers(-(6 << 19), 6 << 19, size=(1, 64, 128, 1024), dtype=np.int64)
        leg("softmax_q19", lambda: oracle.softmax_q19(xs), xs.size, "rows of config 3: [1,64,128,1024]")
        xa = rng.integers(-(16 << 23), 16 << 23, size=(1, 512, 18432), dtype=np.int64)
        leg("silu_q23", lambda: oracle.silu_q23(xa), xa.size, "[1,512,18432]")
        leg("sigmoid_q23", lambda: oracle.sigmoid_q23(xa), xa.size, "[1,512,18432]")
        xr = rng.integers(-(1 << 37), 1 << 37, size=(2048, 7168), dtype=np.int64)
        wr = rng.integers(1 << 18, 1 << 20, size=(7168,), dtype=np.int64).astype(np.int32)
        leg("rmsnorm", lambda: oracle.RMS_Norm_int64(xr, wr, 1, 7168), xr.size, "[2048,7168], int32 weights")
        oracle.set_threads(1)
        res["fixed_point_kernels"] = others
    except Exception as e:                                  # the CPU timings are a reported baseline, never a reason to fail
        res["fixed_point_kernels"] = {"error": repr(e)}
    return res


if __name__ == "__main__":
    main()
