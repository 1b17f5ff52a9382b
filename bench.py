"""Headline benchmark: Wavefunction Embedding forward at B=1, N=16384, d_model=512
(BASELINE.json configs[1]) on one MI355X.  Beside it, one timed leg per other configuration
(configs[0] WE N=512; configs[2] padded attention B=4 N=4096; configs[3] encoder forward;
configs[4] WE N=65536 and attention N=16384), roofline fractions for every kernel and the
CPU PyTorch path timed on the host cores as a baseline for each.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--legs a,b,...] [--no-cpu] [--full-cpu]

Prints ONE JSON line.  A "step" is one WE forward over the whole batch, inputs
and outputs resident in HBM, outputs pre-allocated.

Counter-derived fields (traffic, mfma_util, valu_insts_per_unit) are read from the rocprofv3
summaries under profiles/ (lines of the form "name = number"); each carries a "source" key.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# published MI355X peaks used as roofline denominators
PEAK_FP32_VECTOR_TFLOPS = 157.3     # packed-FMA vector fp32
PEAK_BF16_MFMA_TFLOPS = 2500.0      # dense bf16 matrix
PEAK_HBM_GBS = 8000.0               # HBM3E
H100_REFERENCE_GPW = 6.87194767e10 / 0.386 / 1e9   # README.md:34: 386 ms at this exact shape on an H100

LEGS = ("we_lean", "we_bwd", "aniso", "cfg1", "cfg3", "cfg5_we", "attn", "attn_bwd", "encoder")
PROFILE_WE = "profiles/we_fwd_N16384_K256__counters.txt"
PROFILE_ATTN = "profiles/geo_attn_fwd_N16384_H8_d64__counters.txt"
PROFILE_ATTN_BWD = "profiles/geo_attn_bwd_N16384_H8_d64__counters.txt"


def read_profile(rel):
    """{name: float} from the 'name = number' lines of a summary under profiles/ ({} if the file is absent)."""
    vals = {}
    try:
        with open(os.path.join(ROOT, rel)) as f:
            for line in f:
                m = re.match(r"^\s*([A-Za-z_][A-Za-z0-9_.]*)\s*=\s*([-+0-9.eE]+)\s*(#.*)?$", line)
                if m:
                    vals[m.group(1)] = float(m.group(2))
    except OSError:
        pass
    return vals


def traffic_from(rel):
    """HBM bytes per launch from FETCH_SIZE / WRITE_SIZE (KiB per dispatch) and the copy-kernel calibration factors."""
    p = read_profile(rel)
    need = ("FETCH_SIZE_KiB", "FETCH_SIZE_scale", "WRITE_SIZE_KiB", "WRITE_SIZE_scale")
    if not all(k in p for k in need):
        return None, None
    return int((p["FETCH_SIZE_KiB"] * p["FETCH_SIZE_scale"] + p["WRITE_SIZE_KiB"] * p["WRITE_SIZE_scale"]) * 1024), rel


def settle(torch, fn, min_ms=60.0):
    """Run fn untimed for at least min_ms: while a leg's inputs are made on the host the GPU idles and drops its
    clocks, and the first ~25 ms of work afterwards run below the sustained rate."""
    t0 = time.perf_counter()
    while True:
        fn()
        torch.cuda.synchronize()
        if (time.perf_counter() - t0) * 1e3 >= min_ms:
            break


def time_launches(torch, fn, n, min_settle_ms=60.0):
    """(mean ms, median ms) of n launches of fn, each bracketed by events on torch's current stream (the stream every
    leg passes to the library)."""
    settle(torch, fn, min_settle_ms)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for e0, e1 in ev:
        e0.record()
        fn()
        e1.record()
    torch.cuda.synchronize()
    ms = sorted(e0.elapsed_time(e1) for e0, e1 in ev)
    return sum(ms) / n, ms[n // 2]


def cpu_timed(fn, budget_s, max_runs):
    """Median wall time of up to max_runs runs of fn, stopping once budget_s is spent (always at least one run)."""
    times, spent = [], 0.0
    while len(times) < max_runs and (not times or spent + times[-1] <= budget_s):
        t = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t)
        spent += times[-1]
    times.sort()
    return times[len(times) // 2], len(times)


def probe_rates(lib, torch, dev):
    """Measured lane-op rates (lane-ops/s) of the instructions the WE inner loop issues."""
    # scalar-operand forms (ops 0-2), transcendentals, and the vector-operand forms of the accumulations
    names = {0: "fma_s", 1: "mul_s", 2: "add_s", 3: "sin", 4: "cos", 5: "exp2", 6: "rsq", 7: "fract",
             8: "fmac_v", 9: "add_v"}
    sink = torch.empty(2048 * 256, device=dev)
    rates = {}
    for op, name in names.items():
        blocks, iters = 2048, 1000
        lib.proteus_probe_valu_rate(op, blocks, iters, sink.data_ptr(), None)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        lib.proteus_probe_valu_rate(op, blocks, iters, sink.data_ptr(), None)
        e1.record()
        torch.cuda.synchronize()
        rates[name] = blocks * 256 * iters * 64 / (e0.elapsed_time(e1) * 1e-3)
    return rates


def probe_trans_valu_overlap(lib, torch, dev, waves_per_simd=3, blocks=256):
    """Do transcendental and ordinary vector instructions of different waves of one SIMD overlap?

    One workgroup per compute unit, `waves_per_simd` waves on every SIMD (the headline kernel's occupancy), k of them
    issuing only v_sin_f32 chains and the others only v_fmac_f32 chains with vector-register operands; iteration counts
    chosen so that either group alone takes about the same time.  Returns per k: the two times alone, the time
    together, and hidden = (alone_t + alone_v - together) / min(alone_t, alone_v): 0 = they take turns, 1 = the shorter
    runs entirely beside the longer.  The placement (waves_per_simd waves of a workgroup on each SIMD) is read back
    from the hardware-id register and reported."""
    sink = torch.empty(blocks * 256 * waves_per_simd, device=dev)
    census = torch.zeros(blocks * 4, dtype=torch.int32, device=dev)

    def run(k, it_t, it_v):
        def go():
            rc = lib.proteus_probe_trans_valu_mix(waves_per_simd, k, blocks, it_t, it_v, sink.data_ptr(), census.data_ptr(), None)
            assert rc == 0, rc
        go()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            go()
            e1.record()
            torch.cuda.synchronize()
            best = e0.elapsed_time(e1) if best is None else min(best, e0.elapsed_time(e1))
        return best

    out = {"waves_per_simd": waves_per_simd}
    base = 4000
    for k in range(1, waves_per_simd):
        # calibrate: links of the ordinary group so that it takes as long alone as the transcendental group alone
        t_alone = run(k, base, 0)
        v_probe = run(k, 0, base)
        it_v = max(1, int(base * t_alone / v_probe))
        v_alone = run(k, 0, it_v)
        both = run(k, base, it_v)
        cen = census.cpu().numpy().astype("int64")
        placed_ok = bool(((cen >> 16) == waves_per_simd).all() and ((cen & 0xffff) == k).all())
        out[f"k{k}"] = {
            "trans_waves": k, "valu_waves": waves_per_simd - k, "trans_alone_ms": t_alone, "valu_alone_ms": v_alone,
            "together_ms": both, "hidden": (t_alone + v_alone - both) / min(t_alone, v_alone),
            "placement_as_assumed": placed_ok,
            "lane_ops_per_s_together": {"transcendental": blocks * 4 * k * 64.0 * base * 64 / (both * 1e-3),
                                        "ordinary": blocks * 4 * (waves_per_simd - k) * 64.0 * it_v * 64 / (both * 1e-3)},
        }
    return out


def probe_slot_ms(lib, torch, dev, mode, blocks=512, iters=4000):
    """Seconds per slot per SIMD of the co-issue probe (a slot = one 32x32x16 bf16 product + the softmax work of two
    scores) at two waves per SIMD: blocks x 4 waves x iters x 8 slots over 1024 SIMDs."""
    sink = torch.empty(blocks * 256, device=dev)
    lib.proteus_probe_mfma_softmax_slot(mode, blocks, iters, sink.data_ptr(), None)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    lib.proteus_probe_mfma_softmax_slot(mode, blocks, iters, sink.data_ptr(), None)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / (blocks * 4 * iters * 8 / 1024.0)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--legs", default="all", help="comma-separated legs beside the headline one: " + ",".join(LEGS) + ", all, none")
    ap.add_argument("--no-cpu", action="store_true", help="skip every CPU baseline")
    ap.add_argument("--full-cpu", action="store_true",
                    help="run the CPU path of the headline shape (and of the N=16384 attention) in full, once, instead of on a sample of rows")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target duration of the headline CPU baseline sample")
    ap.add_argument("--we-tuning", type=int, default=0)
    ap.add_argument("--copy-calib", action="store_true",
                    help="also launch a 256 MiB device copy, so a rocprofv3 --pmc run of this command holds a kernel of known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (observer rows and (batch, head) pairs are "
              "independent, so the work shards without any exchange); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    legs = set(LEGS) if args.legs == "all" else set() if args.legs == "none" else set(args.legs.split(","))
    unknown = legs - set(LEGS)
    if unknown:
        print(f"unknown legs: {sorted(unknown)}", file=sys.stderr)
        sys.exit(2)

    import torch
    from proteusai_amd import _lib, _probes, synth
    lib = _lib.load()
    probes = _probes.load()                   # measurement-only library (instruction rates, co-issue); not the product
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream().cuda_stream
    threads = torch.get_num_threads()
    if not args.no_cpu:
        from oracle import torch_oracle

    def we_forward_into(c, w, m, out, cs, ss, tuning=0):
        Zc, Nc, _ = c.shape
        rc = lib.proteus_we_fwd(c.data_ptr(), _lib.COORDS_AOS, w.data_ptr(), None if m is None else m.data_ptr(), out.data_ptr(),
                                None if cs is None else cs.data_ptr(), None if ss is None else ss.data_ptr(),
                                Zc, Nc, w.numel(), tuning, stream)
        if rc != 0:
            _lib.check(rc, "proteus_we_fwd")

    # ---------------- WE forward, B=1, N=16384, d_model=512, compacted random-walk chain ----------------
    Z, N, d_model = 1, 16384, 512
    coords, wn = synth.we_inputs(N, seed=2, batch=Z, d_model=d_model, compact=True)
    K = wn.numel()
    c, w = coords.to(dev).contiguous(), wn.to(dev)
    out = torch.empty(Z, N, 2 * K, device=dev)
    cs = torch.empty(Z, N, K, device=dev)
    ss = torch.empty(Z, N, K, device=dev)

    def we_step():
        we_forward_into(c, w, None, out, cs, ss, args.we_tuning)

    for _ in range(args.warmup):
        we_step()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for e0, e1 in evs:
        e0.record()
        we_step()
        e1.record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    kernel_ms = [e0.elapsed_time(e1) for e0, e1 in evs]
    avg_kernel_ms = sum(kernel_ms) / len(kernel_ms)
    ms_per_step = elapsed * 1e3 / args.steps
    W = float(Z) * N * N * K                          # pair*wavenumber evaluations per step
    value = W * args.steps / elapsed / 1e9            # Gpair*wavenumber/s, whole job

    rates = probe_rates(probes, torch, dev)
    # per unit: the phase product (scalar operand), v_sin, v_cos, two v_fmac and two v_add on vector operands
    r_trans = (rates["sin"] + rates["cos"]) / 2
    per_unit_s = 1.0 / rates["mul_s"] + 2.0 / rates["fmac_v"] + 2.0 / rates["add_v"] + 2.0 / r_trans
    t_model_ms = W * per_unit_s * 1e3
    achieved_tflops = 9.0 * W / (avg_kernel_ms * 1e-3) / 1e12   # 9 flop per unit, FMA counted as 2
    we_traffic, we_traffic_src = traffic_from(PROFILE_WE)
    roofline = {
        "kernel": "we_fwd_kernel", "bound": "valu", "achieved": achieved_tflops, "peak": PEAK_FP32_VECTOR_TFLOPS,
        "unit": "TFLOP/s", "frac": achieved_tflops / PEAK_FP32_VECTOR_TFLOPS,
        "traffic": we_traffic, "traffic_source": we_traffic_src,
        "kernel_ms": avg_kernel_ms,
        "issue_model": {
            "lane_ops_per_unit": {"mul_scalar_operand": 1, "fmac_vector_operands": 2, "add_vector_operands": 2,
                                  "transcendental": 2},
            "measured_lane_ops_per_s": {"mul_scalar_operand": rates["mul_s"], "fmac_vector_operands": rates["fmac_v"],
                                        "add_vector_operands": rates["add_v"], "transcendental": r_trans},
            "model_ms": t_model_ms, "frac": t_model_ms / avg_kernel_ms,
        },
        # the same model with the vendor-derived rates instead of the measured ones: 256 CUs x 4 SIMDs x 16 lanes x
        # 2.4 GHz for the five ordinary operations, a quarter of that for the two transcendentals
        "vendor_rate_model": {"lane_ops_per_s": {"ordinary": 3.93e13, "transcendental": 9.83e12},
                              "model_ms": W * (5.0 / 3.93e13 + 2.0 / 9.83e12) * 1e3,
                              "frac": W * (5.0 / 3.93e13 + 2.0 / 9.83e12) * 1e3 / avg_kernel_ms},
    }
    # the published 157.3 TFLOP/s counts packed (two-wide) fp32 FMAs, which this build never issues; beside it the
    # fraction of the one-wide vector rate, half of it
    roofline["peak_non_packed"] = PEAK_FP32_VECTOR_TFLOPS / 2
    roofline["frac_of_non_packed_peak"] = achieved_tflops / (PEAK_FP32_VECTOR_TFLOPS / 2)
    # The issue model adds the transcendentals' time to the ordinary instructions' time.  Whether the two kinds, issued
    # by different waves of a SIMD, run beside each other is measured here; if they did, the bound would be the larger
    # of the two times instead of their sum.
    t_ord_ms = W * (1.0 / rates["mul_s"] + 2.0 / rates["fmac_v"] + 2.0 / rates["add_v"]) * 1e3
    t_trn_ms = W * (2.0 / r_trans) * 1e3
    overlap = probe_trans_valu_overlap(probes, torch, dev)
    hidden = min(v["hidden"] for k_, v in overlap.items() if k_.startswith("k"))
    hidden = max(0.0, min(1.0, hidden))
    bound_ms = t_ord_ms + t_trn_ms - hidden * min(t_ord_ms, t_trn_ms)
    roofline["issue_model"]["trans_valu_overlap"] = {
        "probe": overlap, "hidden_fraction_used": hidden,
        "ordinary_ms": t_ord_ms, "transcendental_ms": t_trn_ms,
        "model_ms_with_measured_overlap": bound_ms, "frac_with_measured_overlap": bound_ms / avg_kernel_ms,
        "model_ms_if_fully_overlapped": max(t_ord_ms, t_trn_ms), "frac_if_fully_overlapped": max(t_ord_ms, t_trn_ms) / avg_kernel_ms,
    }
    pw = read_profile(PROFILE_WE)
    if "valu_insts_per_unit" in pw:
        roofline["valu_insts_per_unit"] = {
            "value": pw["valu_insts_per_unit"], "add_f32": pw.get("add_f32_per_unit"), "mul_f32": pw.get("mul_f32_per_unit"),
            "fma_f32": pw.get("fma_f32_per_unit"), "trans_f32": pw.get("trans_f32_per_unit"),
            "valu_active_frac": pw.get("valu_active_frac"), "source": PROFILE_WE}

    result = {
        "metric": "we_fwd_gpair_wavenumber_per_s", "value": value, "unit": "Gpair*wavenumber/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": value / H100_REFERENCE_GPW,
        "baseline_note": "reference README.md:34: 386 ms (178 Gpair*wavenumber/s) for this shape on an H100",
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "WE forward B=1 N=16384 d_model=512 (256 wavenumbers), compacted random-walk C-alpha chain, "
                               "lambda 3.7-20 A base 20, no mask (BASELINE.json configs[1])",
                   "Z": Z, "N": N, "K": K, "we_variant": _lib.we_variants()[args.we_tuning]},
        "roofline": roofline,
    }

    def we_model_frac(units, ms):
        return units * per_unit_s * 1e3 / ms

    # ---------------- the same forward without the cos/sin sums (inference: nothing kept for a backward) ----------
    if "we_lean" in legs:
        lean_ms, _ = time_launches(torch, lambda: we_forward_into(c, w, None, out, None, None, args.we_tuning), max(5, args.steps // 2), 0.0)
        # per unit: the phase product, v_sin, v_cos and two v_fmac (the two v_add of the plain sums are gone)
        lean_model_ms = W * (1.0 / rates["mul_s"] + 2.0 / rates["fmac_v"] + 2.0 / r_trans) * 1e3
        result["we_fwd_without_sums"] = {
            "workload": "the headline shape with cos_sums = sin_sums = NULL (embedding only; not the headline metric, "
                        "whose forward also returns the sums as the reference's does)",
            "ms": lean_ms, "gpair_wavenumber_per_s": W / (lean_ms * 1e-3) / 1e9, "dtype": "f32",
            "issue_model": {"model_ms": lean_model_ms, "frac": lean_model_ms / lean_ms},
        }

    # ---------------- WE backward (the reduction of dO against the sums), same shape: HBM-bound ----------------
    if "we_bwd" in legs:
        dO = torch.randn(Z, N, 2 * K, device=dev)
        dk = torch.empty(K, device=dev)
        ws_bytes = lib.proteus_we_bwd_workspace_bytes(Z, N, K)
        ws = torch.empty(ws_bytes // 4, device=dev)

        def we_bwd_step():
            rc = lib.proteus_we_bwd(dO.data_ptr(), cs.data_ptr(), ss.data_ptr(), dk.data_ptr(), ws.data_ptr(), ws_bytes,
                                    Z, N, K, stream)
            if rc != 0:
                _lib.check(rc, "proteus_we_bwd")
        _, b_ms = time_launches(torch, we_bwd_step, 20)
        b_bytes = 16.0 * Z * N * K                       # dO (8) + cos_sums (4) + sin_sums (4) per (token, wavenumber)
        result["we_bwd"] = {
            "workload": "WE backward for the wavenumbers, dO [1,16384,512] against the saved sums, two launches",
            "ms": b_ms, "dtype": "f32",
            "roofline": {"kernel": "we_bwd_partial_kernel + we_bwd_final_kernel", "bound": "hbm",
                         "achieved": b_bytes / (b_ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": b_bytes / (b_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, "traffic": None},
        }
        del dO, ws

    # ---------------- anisotropic (C-beta scaled) WE forward, same shape and chain ----------------
    if "aniso" in legs:
        g = torch.Generator().manual_seed(2)
        cbv = torch.randn(Z, N, 3, generator=g)
        cbv = (cbv / cbv.norm(dim=-1, keepdim=True)).to(dev).contiguous()
        cbm = (0.5 + 2.0 * torch.rand(K, generator=g)).to(dev)
        ao = [torch.empty(Z, N, 2 * K, device=dev) for _ in range(3)]

        def aniso_step():
            rc = lib.proteus_we_aniso_fwd(c.data_ptr(), cbv.data_ptr(), _lib.COORDS_AOS, cbm.data_ptr(), w.data_ptr(), None,
                                          ao[0].data_ptr(), ao[1].data_ptr(), ao[2].data_ptr(), Z, N, K, 0, stream)
            if rc != 0:
                _lib.check(rc, "proteus_we_aniso_fwd")
        x_ms, _ = time_launches(torch, aniso_step, max(5, args.steps // 2), 0.0)
        # per unit: 2 scalar-operand phase ops, 4 v_fmac + 2 v_add on vector operands, v_sin, v_cos (no v_fract: at this
        # shape every phase provably stays within the range the two accept)
        x_model_ms = W * (2.0 / rates["mul_s"] + 4.0 / rates["fmac_v"] + 2.0 / rates["add_v"] + 2.0 / r_trans) * 1e3
        result["we_aniso"] = {
            "workload": "anisotropic (C-beta scaled) WE forward, out + d_cb + d_k, B=1 N=16384 256 wavenumbers, same chain, random unit C-beta vectors",
            "ms": x_ms, "gpair_wavenumber_per_s": W / (x_ms * 1e-3) / 1e9, "dtype": "f32",
            "issue_model": {"lane_ops_per_unit": {"scalar_operand": 2, "fmac_vector_operands": 4,
                                                  "add_vector_operands": 2, "transcendental": 2},
                            "model_ms": x_model_ms, "frac": x_model_ms / x_ms},
        }

        def aniso_lean_step():
            rc = lib.proteus_we_aniso_fwd(c.data_ptr(), cbv.data_ptr(), _lib.COORDS_AOS, cbm.data_ptr(), w.data_ptr(), None,
                                          ao[0].data_ptr(), None, None, Z, N, K, 0, stream)
            if rc != 0:
                _lib.check(rc, "proteus_we_aniso_fwd")
        xl_ms, _ = time_launches(torch, aniso_lean_step, max(5, args.steps // 2), 0.0)
        result["we_aniso"]["ms_embedding_only"] = xl_ms           # d_cb = d_k = NULL: two running sums per wavenumber instead of six
        del ao

    # ---------------- configs[0]: WE forward B=1, N=512 (the reference's CPU-runnable case) ----------------
    if "cfg1" in legs:
        c1, _ = synth.we_inputs(512, seed=1, batch=1, d_model=d_model, compact=False)
        c1d = c1.to(dev).contiguous()
        o1, cs1, ss1 = (torch.empty(1, 512, n, device=dev) for n in (2 * K, K, K))
        _, ms1 = time_launches(torch, lambda: we_forward_into(c1d, w, None, o1, cs1, ss1), 200)
        W1 = 512.0 * 512 * K
        leg = {"workload": "WE forward B=1 N=512 d_model=512, random-walk chain, no mask (BASELINE.json configs[0]); "
                           "8 observer blocks of 64 rows x 64 tiles of 4 wavenumbers: 512 short workgroups, a launch-latency-sized kernel",
               "ms": ms1, "gpair_wavenumber_per_s": W1 / (ms1 * 1e-3) / 1e9, "dtype": "f32",
               "roofline": {"kernel": "we_fwd_kernel", "bound": "valu", "achieved": 9.0 * W1 / (ms1 * 1e-3) / 1e12,
                            "peak": PEAK_FP32_VECTOR_TFLOPS, "unit": "TFLOP/s",
                            "frac": 9.0 * W1 / (ms1 * 1e-3) / 1e12 / PEAK_FP32_VECTOR_TFLOPS,
                            "issue_model_frac": we_model_frac(W1, ms1)}}
        if not args.no_cpu:
            dt, runs = cpu_timed(lambda: torch_oracle.we_torch(c1, wn), 10.0, 5)
            leg["cpu_baseline"] = {"value": W1 / dt / 1e9, "unit": "Gpair*wavenumber/s", "cores": threads, "kind": "port",
                                   "sample": f"the full workload, median of {runs} runs, tiled CPU PyTorch fp32, {dt * 1e3:.1f} ms"}
        result["cfg1_we_n512"] = leg

    # ---------------- configs[4], WE half: B=1, N=65536, same compacted-chain generator ----------------
    if "cfg5_we" in legs:
        c5, _ = synth.we_inputs(65536, seed=5, compact=True)
        c5d = c5.to(dev).contiguous()
        o5, cs5, ss5 = (torch.empty(1, 65536, n, device=dev) for n in (2 * K, K, K))
        ms5, _ = time_launches(torch, lambda: we_forward_into(c5d, w, None, o5, cs5, ss5), 3, 0.0)
        W5 = 65536.0 * 65536 * K
        leg = {"workload": "WE forward B=1 N=65536 d_model=512, compacted random-walk chain, no mask (BASELINE.json configs[4])",
               "ms": ms5, "gpair_wavenumber_per_s": W5 / (ms5 * 1e-3) / 1e9, "dtype": "f32",
               "roofline": {"kernel": "we_fwd_kernel", "bound": "valu", "achieved": 9.0 * W5 / (ms5 * 1e-3) / 1e12,
                            "peak": PEAK_FP32_VECTOR_TFLOPS, "unit": "TFLOP/s",
                            "frac": 9.0 * W5 / (ms5 * 1e-3) / 1e12 / PEAK_FP32_VECTOR_TFLOPS,
                            "issue_model_frac": we_model_frac(W5, ms5)}}
        if not args.no_cpu:
            sel = torch.linspace(0, 65535, 256).long().tolist()
            t = time.perf_counter()
            torch_oracle.we_torch(c5, wn, rows=sel)
            dt = time.perf_counter() - t
            leg["cpu_baseline"] = {"value": 256 * 65536.0 * K / dt / 1e9, "unit": "Gpair*wavenumber/s", "cores": threads,
                                   "kind": "port", "extrapolated": True,
                                   "sample": f"256 of 65536 observer rows (all 65536 sources each), tiled CPU PyTorch fp32, {dt:.1f} s; "
                                             f"the full workload at this rate: {dt * 256:.0f} s"}
        result["cfg5_we_n65536"] = leg
        del o5, cs5, ss5, c5d

    def attn_forward_into(q, k, v, cd, sg, m, O, L):
        Za, Ha, Na, da = q.shape
        rc = lib.proteus_geo_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), cd.data_ptr(), sg.data_ptr(),
                                      None if m is None else m.data_ptr(), O.data_ptr(), L.data_ptr(), Za, Ha, Na, da, 0, stream)
        if rc != 0:
            _lib.check(rc, "proteus_geo_attn_fwd")

    # ---------------- configs[2]: geometric attention B=4, N=4096, H=8, d=64, lengths in [2048, 4096] ----------------
    if "cfg3" in legs:
        Q3, K3, V3, c3, sg3, m3 = synth.attn_inputs(4, 8, 4096, 64, seed=3, min_len=2048)
        q3, k3, v3, c3d, s3d, m3d = (t.to(dev) for t in (Q3, K3, V3, c3, sg3, m3))
        O3 = torch.empty(4, 8, 4096, 64, device=dev)
        L3 = torch.empty(4, 8, 4096, device=dev)
        # the entry point with a caller-provided workspace (allocated once, outside the timed region, like the outputs):
        # with it the library runs padded batches on the balanced schedule
        ws3_bytes = lib.proteus_geo_attn_fwd_workspace_bytes(4, 8, 4096, 64, 0)
        ws3 = torch.empty(max(ws3_bytes, 256), dtype=torch.uint8, device=dev)
        m3u = m3d.view(torch.uint8)

        def attn3_step():
            rc = lib.proteus_geo_attn_fwd_ws(q3.data_ptr(), k3.data_ptr(), v3.data_ptr(), None, c3d.data_ptr(), s3d.data_ptr(),
                                             m3u.data_ptr(), O3.data_ptr(), L3.data_ptr(), ws3.data_ptr(), ws3_bytes,
                                             4, 8, 4096, 64, 0, stream)
            if rc != 0:
                _lib.check(rc, "proteus_geo_attn_fwd_ws")
        _, ms3 = time_launches(torch, attn3_step, 50)
        _, ms3_plain = time_launches(torch, lambda: attn_forward_into(q3, k3, v3, c3d, s3d, m3d, O3, L3), 50)

        def attn3_balanced_step():          # the other schedule for padded batches (equal shares of steps, persistent grid)
            rc = lib.proteus_geo_attn_fwd_ws(q3.data_ptr(), k3.data_ptr(), v3.data_ptr(), None, c3d.data_ptr(), s3d.data_ptr(),
                                             m3u.data_ptr(), O3.data_ptr(), L3.data_ptr(), ws3.data_ptr(), ws3_bytes,
                                             4, 8, 4096, 64, 8, stream)
            if rc != 0:
                _lib.check(rc, "proteus_geo_attn_fwd_ws")
        _, ms3_balanced = time_launches(torch, attn3_balanced_step, 50)
        lens = (~m3).sum(dim=1).double()
        useful = 4.0 * 8 * 64 * float((lens * lens).sum())
        dense = 4.0 * 4 * 8 * 64 * 4096 * 4096
        leg = {"workload": "geometric attention forward B=4 H=8 N=4096 d_head=64 bf16, random-walk chains, sigma 3-25 A, "
                           "valid lengths uniform in [2048, 4096], the rest padded (BASELINE.json configs[2])",
               "ms": ms3, "lengths": [int(x) for x in lens], "dtype": "bf16",
               "tflops_useful": useful / (ms3 * 1e-3) / 1e12, "tflops_dense_equivalent": dense / (ms3 * 1e-3) / 1e12,
               "entry_point": "proteus_geo_attn_fwd_ws (plan kernel + split-items grid: two launches)",
               "ms_plain_grid": ms3_plain, "ms_balanced_schedule": ms3_balanced,
               "roofline": {"kernel": "geo_attn_plan_kernel + geo_attn_fwd_split_kernel",
                            "bound": "mfma", "achieved": useful / (ms3 * 1e-3) / 1e12,
                            "peak": PEAK_BF16_MFMA_TFLOPS, "unit": "TFLOP/s",
                            "frac": useful / (ms3 * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS,
                            "frac_plain_grid": useful / (ms3_plain * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS,
                            "flop": "4 H d sum_b L_b^2 (pairs of valid tokens only)"}}
        # the backward of the same padded batch (kernel call only: D precomputed; d_sigma accumulates, it is not read)
        attn_forward_into(q3, k3, v3, c3d, s3d, m3d, O3, L3)
        g3 = torch.Generator().manual_seed(3)
        dO3 = (torch.randn(4, 8, 4096, 64, generator=g3) / 8).bfloat16().to(dev)
        D3 = (O3 * dO3.float()).sum(-1).contiguous()
        dQ3, dK3, dV3 = (torch.empty(4, 8, 4096, 64, device=dev) for _ in range(3))
        ds3 = torch.zeros(8, device=dev)

        def bwd3_step():
            rc = lib.proteus_geo_attn_bwd(q3.data_ptr(), k3.data_ptr(), v3.data_ptr(), dO3.data_ptr(), c3d.data_ptr(), s3d.data_ptr(),
                                          None, m3d.data_ptr(), L3.data_ptr(), D3.data_ptr(), dQ3.data_ptr(), dK3.data_ptr(), dV3.data_ptr(),
                                          ds3.data_ptr(), None, 4, 8, 4096, 64, 0.0, 1.0, _lib.OPERAND_BF16, stream)
            if rc != 0:
                _lib.check(rc, "proteus_geo_attn_bwd")
        _, bms3 = time_launches(torch, bwd3_step, 20)
        leg["backward_ms"] = bms3
        leg["backward_tflops_useful_5_products"] = 2.5 * useful / (bms3 * 1e-3) / 1e12
        leg["backward_frac"] = 2.5 * useful / (bms3 * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS
        del dO3, D3, dQ3, dK3, dV3
        if not args.no_cpu:
            dt, runs = cpu_timed(lambda: torch_oracle.geo_attn_torch(Q3, K3, V3, c3, sg3, m3), 20.0, 3)
            leg["cpu_baseline"] = {"value": dense / dt / 1e12, "unit": "TFLOP/s (dense-equivalent: the CPU path computes every pair and masks)",
                                   "cores": threads, "kind": "port",
                                   "sample": f"the full workload, median of {runs} run(s), dense CPU PyTorch fp32 on the bf16-rounded inputs, {dt:.1f} s"}
        result["cfg3_attn_b4_n4096_padded"] = leg
        del q3, k3, v3, O3, L3, ws3

    # ---------------- one unpadded sequence that does not fill the chip: Z=1, H=8, N=8192 (not a BASELINE configuration) ----------------
    if "attn" in legs:
        Q1, K1, V1, c1, sg1, _ = synth.attn_inputs(1, 8, 8192, 64, seed=8)
        q1, k1, v1, c1d, s1d = (t.to(dev) for t in (Q1, K1, V1, c1, sg1))
        O1 = torch.empty(1, 8, 8192, 64, device=dev)
        L1 = torch.empty(1, 8, 8192, device=dev)
        ws1_bytes = lib.proteus_geo_attn_fwd_workspace_bytes(1, 8, 8192, 64, 0)
        ws1 = torch.empty(max(ws1_bytes, 256), dtype=torch.uint8, device=dev)

        def attn1_step():
            rc = lib.proteus_geo_attn_fwd_ws(q1.data_ptr(), k1.data_ptr(), v1.data_ptr(), None, c1d.data_ptr(), s1d.data_ptr(),
                                             None, O1.data_ptr(), L1.data_ptr(), ws1.data_ptr(), ws1_bytes, 1, 8, 8192, 64, 0, stream)
            if rc != 0:
                _lib.check(rc, "proteus_geo_attn_fwd_ws")
        _, ms1 = time_launches(torch, attn1_step, 30)
        _, ms1_plain = time_launches(torch, lambda: attn_forward_into(q1, k1, v1, c1d, s1d, None, O1, L1), 30)
        flop1 = 4.0 * 8 * 64 * 8192.0 * 8192.0
        result["geo_attn_single_sequence_n8192"] = {
            "workload": "geometric attention forward Z=1 H=8 N=8192 d_head=64 bf16, no mask: 256 items for 512 workgroup slots "
                        "(with a workspace every item is split into two parts)",
            "ms": ms1, "ms_plain_grid": ms1_plain, "tflops": flop1 / (ms1 * 1e-3) / 1e12,
            "frac": flop1 / (ms1 * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS,
            "frac_plain_grid": flop1 / (ms1_plain * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS}
        del q1, k1, v1, O1, L1, ws1

    # ---------------- geometric attention forward, N=16384, H=8, d=64 (configs[4]) ----------------
    if "attn" in legs or "attn_bwd" in legs:
        wc, _ = synth.we_inputs(65536, seed=5, compact=True)
        Q, Kt, V, ac, sigma, _ = synth.attn_inputs(1, 8, 16384, 64, seed=5, coords=wc[:, :16384].contiguous())
        q, k, v, acd, sg = Q.to(dev), Kt.to(dev), V.to(dev), ac.to(dev), sigma.to(dev)
        O = torch.empty(1, 8, 16384, 64, device=dev)
        L = torch.empty(1, 8, 16384, device=dev)
        a_ms, _ = time_launches(torch, lambda: attn_forward_into(q, k, v, acd, sg, None, O, L), max(10, args.steps))
        flops = 4.0 * 8 * 64 * 16384 * 16384
        a_tflops = flops / (a_ms * 1e-3) / 1e12
        a_traffic, a_traffic_src = traffic_from(PROFILE_ATTN)
        leg = {
            "workload": "geometric attention forward Z=1 H=8 N=16384 d_head=64 bf16, compacted chain, sigma 3-25 A (BASELINE.json configs[4])",
            "ms": a_ms, "tflops": a_tflops, "dtype": "bf16",
            "roofline": {"kernel": "geo_attn_fwd_pipe_kernel", "bound": "mfma", "achieved": a_tflops, "peak": PEAK_BF16_MFMA_TFLOPS,
                         "unit": "TFLOP/s", "frac": a_tflops / PEAK_BF16_MFMA_TFLOPS,
                         "traffic": a_traffic, "traffic_source": a_traffic_src},
        }
        # Issue model: the kernel's inner loop is eight "slots" per 32 x 32 block of pairs (8 matrix products: 4 for the
        # scores, 4 for P V), each with the softmax work of two scores per lane.  The probe measures what one SIMD needs per
        # slot at the kernel's occupancy (two waves) when it does nothing else: no staging, no geometry, no barrier.
        slots = 8.0 * 8 * (16384 / 32) * (16384 / 32) / 1024.0               # per SIMD
        t_m, t_v, t_b = (probe_slot_ms(probes, torch, dev, m) for m in (0, 1, 2))
        leg["roofline"]["issue_model"] = {
            "slot": "one 32x32x16 bf16 product + 2 fma + 2 exp2 + 1 pack + 1 packed add, two waves per SIMD",
            "ns_per_slot_per_simd": {"matrix_only": t_m * 1e9, "vector_only": t_v * 1e9, "both": t_b * 1e9},
            "model_ms": slots * t_b * 1e3, "frac": slots * t_b * 1e3 / a_ms,
            "matrix_only_ms": slots * t_m * 1e3,
        }
        # which vector instructions run beside a matrix product: the same loop with the softmax work replaced by
        # twelve ordinary fused multiply-adds, and by four exp2 (ns per slot and SIMD: alone, and with the product)
        t_pa, t_pm, t_ta, t_tm = (probe_slot_ms(probes, torch, dev, m) for m in (3, 4, 5, 6))
        leg["roofline"]["issue_model"]["beside_a_product_ns"] = {
            "twelve_fma": {"alone": t_pa * 1e9, "with_product": t_pm * 1e9, "hidden_frac": (t_m + t_pa - t_pm) / t_pa},
            "four_exp2": {"alone": t_ta * 1e9, "with_product": t_tm * 1e9, "hidden_frac": (t_m + t_ta - t_tm) / t_ta},
        }
        pa_ = read_profile(PROFILE_ATTN)
        if "mfma_util" in pa_:
            leg["roofline"]["mfma_util"] = {"value": pa_["mfma_util"], "mfma_flop_counted": pa_.get("mfma_flop"),
                                            "lds_wait_frac": pa_.get("lds_wait_frac"), "source": PROFILE_ATTN}
        if not args.no_cpu and "attn" in legs:
            rows = None if args.full_cpu else torch.linspace(0, 16383, 1024).long().tolist()
            t = time.perf_counter()
            torch_oracle.geo_attn_torch(Q, Kt, V, ac, sigma, None, rows=rows)
            dt = time.perf_counter() - t
            n_rows = 16384 if rows is None else len(rows)
            leg["cpu_baseline"] = {"value": flops * n_rows / 16384 / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                                   "extrapolated": rows is not None,
                                   "sample": f"{n_rows} of 16384 query rows of every head (all 16384 keys each), dense CPU PyTorch fp32, {dt:.1f} s"}
        result["geo_attn"] = leg

        # ---- backward of the same shape (dQ, dK, dV, d sigma from the forward's O and L) ----
        if "attn_bwd" in legs:
            gq = torch.Generator().manual_seed(5)
            dOb = (torch.randn(1, 8, 16384, 64, generator=gq) / 8).bfloat16().to(dev)
            Dv = (O * dOb.float()).sum(-1).contiguous()
            dQ_, dK_, dV_ = (torch.empty(1, 8, 16384, 64, device=dev) for _ in range(3))
            dsg = torch.zeros(8, device=dev)

            def bwd_step():
                rc = lib.proteus_geo_attn_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), dOb.data_ptr(), acd.data_ptr(), sg.data_ptr(),
                                              None, None, L.data_ptr(), Dv.data_ptr(), dQ_.data_ptr(), dK_.data_ptr(), dV_.data_ptr(),
                                              dsg.data_ptr(), None, 1, 8, 16384, 64, 0.0, 1.0, _lib.OPERAND_BF16, stream)
                if rc != 0:
                    _lib.check(rc, "proteus_geo_attn_bwd")
            b_ms, _ = time_launches(torch, bwd_step, 5)
            b_traffic, b_traffic_src = traffic_from(PROFILE_ATTN_BWD)
            result["geo_attn_bwd"] = {
                "workload": "geometric attention backward, same shape: dQ, dK, dV, d_sigma (two passes in one launch, S and dP recomputed in each)",
                "ms": b_ms, "tflops_5_products": 10.0 * 8 * 64 * 16384 * 16384 / (b_ms * 1e-3) / 1e12,
                "tflops_issued_7_products": 14.0 * 8 * 64 * 16384 * 16384 / (b_ms * 1e-3) / 1e12, "dtype": "bf16",
                "roofline": {"kernel": "geo_attn_bwd_kernel", "bound": "mfma",
                             "achieved": 10.0 * 8 * 64 * 16384 * 16384 / (b_ms * 1e-3) / 1e12, "peak": PEAK_BF16_MFMA_TFLOPS,
                             "unit": "TFLOP/s", "frac": 10.0 * 8 * 64 * 16384 * 16384 / (b_ms * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS,
                             "traffic": b_traffic, "traffic_source": b_traffic_src},
            }
            # D = rowsum(O * dO), taken before the backward kernel (its `D` argument): one pass over O (fp32) and dO (bf16)
            Dk = torch.empty(1, 8, 16384, device=dev)

            def delta_step():
                rc = lib.proteus_geo_attn_delta(O.data_ptr(), dOb.data_ptr(), None, Dk.data_ptr(), 1, 8, 16384, 64, _lib.DTYPE_BF16, stream)
                if rc != 0:
                    _lib.check(rc, "proteus_geo_attn_delta")
            _, d_ms = time_launches(torch, delta_step, 20)
            d_bytes = 8.0 * 16384 * (64 * 6 + 4)
            result["geo_attn_bwd"]["delta"] = {"kernel": "geo_attn_delta_kernel", "ms": d_ms, "bound": "hbm",
                                               "achieved": d_bytes / (d_ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                               "frac": d_bytes / (d_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                               "equals_torch": bool(torch.allclose(Dk, Dv, rtol=1e-5, atol=1e-6))}
            # ---- the reference kernel's own logits (beta-weighted bias, pair mask) at its module's default rbf range:
            #      key tiles whose pairs are all below min_rbf are skipped ----
            bet = torch.full((8,), 0.5, device=dev)
            dbt = torch.zeros(8, device=dev)
            lo_rbf, hi_rbf = 0.001, 1.0

            def legacy_fwd():
                rc = lib.proteus_geo_attn_legacy_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), acd.data_ptr(), sg.data_ptr(), bet.data_ptr(),
                                                     None, O.data_ptr(), L.data_ptr(), 1, 8, 16384, 64, lo_rbf, hi_rbf,
                                                     _lib.OPERAND_BF16, 0, stream)
                if rc != 0:
                    _lib.check(rc, "proteus_geo_attn_legacy_fwd")

            def legacy_bwd():
                rc = lib.proteus_geo_attn_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), dOb.data_ptr(), acd.data_ptr(), sg.data_ptr(),
                                              bet.data_ptr(), None, L.data_ptr(), Dv.data_ptr(), dQ_.data_ptr(), dK_.data_ptr(), dV_.data_ptr(),
                                              dsg.data_ptr(), dbt.data_ptr(), 1, 8, 16384, 64, lo_rbf, hi_rbf, _lib.OPERAND_BF16, stream)
                if rc != 0:
                    _lib.check(rc, "proteus_geo_attn_bwd")
            lf_ms, _ = time_launches(torch, legacy_fwd, 10)
            Dv = (O * dOb.float()).sum(-1).contiguous()
            lb_ms, _ = time_launches(torch, legacy_bwd, 5)
            result["geo_attn_reference_logits"] = {
                "workload": "the same shape with the reference kernel's logits S + beta*rbf_norm*|S| and pair mask, beta 0.5, "
                            "rbf range [0.001, 1] (the reference module's default), bf16 operands",
                "forward_ms": lf_ms, "backward_ms": lb_ms,
                "note": "pairs below min_rbf are masked, so tiles out of reach are skipped: the time depends on sigma"}
            del dOb, Dv, dQ_, dK_, dV_, bet, dbt
        del q, k, v, O, L

    # ---------------- encoder forward, B=8, N=1024, 4 layers, bf16 weights, fp32 WE (configs[3]) ----------------
    if "encoder" in legs:
        import proteusai_amd as pa
        torch.manual_seed(4)
        model = pa.ProteusEncoder().eval()
        state = {k_: v_.clone() for k_, v_ in model.state_dict().items()}
        min_spread = model.layers[0].attn.min_spread
        model.to(dev)
        model.aa_embedding.to(torch.bfloat16)
        model.layers.to(torch.bfloat16)
        model.head.to(torch.bfloat16)
        g = torch.Generator().manual_seed(4)
        ecoords_h = torch.stack([synth.random_walk_chain(1024, g) for _ in range(8)])
        etokens_h = torch.randint(0, 33, (8, 1024), generator=g)
        lens = torch.randint(128, 1025, (8,), generator=g)
        emask_h = torch.arange(1024)[None, :] >= lens[:, None]
        ecoords, etokens, emask = ecoords_h.to(dev), etokens_h.to(dev), emask_h.to(dev)
        with torch.no_grad():
            settle(torch, lambda: model(ecoords, etokens, emask))
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(10):
                model(ecoords, etokens, emask)
            e1.record()
            torch.cuda.synchronize()
        result["encoder_forward"] = {
            "workload": "WE + 33x512 embedding, 4 x (geometric MHA H=8 + LN + FFN 512-2048-512 GELU + LN), head to 20; "
                        "B=8 N=1024 lengths 128-1024, bf16 weights, fp32 WE (BASELINE.json configs[3])",
            "ms": e0.elapsed_time(e1) / 10, "valid_tokens": int(lens.sum()),
            "tokens_per_s": float(lens.sum()) / (e0.elapsed_time(e1) / 10 * 1e-3),
        }
        # the same forward captured into a HIP graph and replayed: what the launches cost goes away
        with torch.no_grad():
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                model(ecoords, etokens, emask)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                graph_out = model(ecoords, etokens, emask)
            torch.cuda.synchronize()
            eager_out = model(ecoords, etokens, emask)
            graph.replay()
            torch.cuda.synchronize()
            same = bool(torch.equal(graph_out[~emask], eager_out[~emask]))
            settle(torch, graph.replay)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(10):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
        result["encoder_forward"]["ms_graph_replay"] = e0.elapsed_time(e1) / 10
        result["encoder_forward"]["graph_replay_equals_eager"] = same
        del graph, graph_out
        if not args.no_cpu:
            with torch.no_grad():
                dt, runs = cpu_timed(lambda: torch_oracle.encoder_forward_torch(state, min_spread, ecoords_h, etokens_h, emask_h), 20.0, 3)
            result["encoder_forward"]["cpu_baseline"] = {
                "value": float(lens.sum()) / dt, "unit": "valid tokens/s", "cores": threads, "kind": "port",
                "sample": f"the full workload, median of {runs} run(s), the same weights in fp32 on the CPU PyTorch path, {dt:.1f} s"}
        # forward + backward of the same stack (cross-entropy on the unpadded tokens), no optimiser step
        model.train()
        labels = torch.randint(0, 20, (8, 1024), generator=g).to(dev)
        keep = ~emask

        def train_step():
            model.zero_grad(set_to_none=True)
            logits = model(ecoords, etokens, emask)
            torch.nn.functional.cross_entropy(logits[keep].float(), labels[keep]).backward()
        settle(torch, train_step)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            train_step()
        e1.record()
        torch.cuda.synchronize()
        result["encoder_forward_backward"] = {"workload": "the same stack and batch, forward + backward (dropout 0)",
                                              "ms": e0.elapsed_time(e1) / 10}

        # the layer's fused residual add + LayerNorm on its own: at the encoder's shape and at a size HBM can show
        lnr = {}
        for rows_ln, tag in ((8 * 1024, "encoder_shape"), (256 * 1024, "large")):
            xa = torch.randn(rows_ln, 512, device=dev).bfloat16()
            xb = torch.randn(rows_ln, 512, device=dev).bfloat16()
            ga, be = torch.ones(512, device=dev).bfloat16(), torch.zeros(512, device=dev).bfloat16()
            xo = torch.empty_like(xa)

            def ln_step():
                rc = lib.proteus_add_layernorm_fwd(xa.data_ptr(), xb.data_ptr(), ga.data_ptr(), be.data_ptr(), xo.data_ptr(),
                                                   rows_ln, 512, 1e-5, _lib.DTYPE_BF16, stream)
                if rc != 0:
                    _lib.check(rc, "proteus_add_layernorm_fwd")
            _, ln_ms = time_launches(torch, ln_step, 20)
            ln_bytes = 3.0 * 2 * rows_ln * 512                 # x, res in; out: bf16
            lnr[tag] = {"rows": rows_ln, "ms": ln_ms, "GB_per_s": ln_bytes / (ln_ms * 1e-3) / 1e9}
            del xa, xb, xo
        result["add_layernorm"] = {
            "workload": "residual add + LayerNorm over 512 features, bf16 (the encoder layer's two normalisations; inference path)",
            "dtype": "bf16", **lnr,
            "roofline": {"kernel": "add_layernorm_kernel", "bound": "hbm", "achieved": lnr["large"]["GB_per_s"], "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": lnr["large"]["GB_per_s"] / PEAK_HBM_GBS, "traffic": None},
        }

    # ---------------- CPU baseline of the headline shape: the tiled CPU PyTorch path on a bounded sample of observer rows --------
    if not args.no_cpu:
        if args.full_cpu:
            rows, sel = N, None
        else:
            rows = 64
            t = time.perf_counter()
            torch_oracle.we_torch(coords, wn, rows=list(range(rows)))
            dt = time.perf_counter() - t
            rows = int(max(64, min(N, rows * args.cpu_seconds / max(dt, 1e-3))))
            rows -= rows % 64
            sel = torch.linspace(0, N - 1, rows).long().tolist()
        t = time.perf_counter()
        torch_oracle.we_torch(coords, wn, rows=sel)
        dt = time.perf_counter() - t
        result["cpu_baseline"] = {
            "value": rows * float(N) * K / dt / 1e9, "unit": "Gpair*wavenumber/s", "cores": threads, "kind": "port",
            "sample": f"{rows} of {N} observer rows of the same workload (all {N} sources each), tiled CPU PyTorch fp32, {dt:.1f} s",
            "host_cpus": os.cpu_count(),
        }

    if args.copy_calib:
        a = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()

    print(json.dumps(result))


if __name__ == "__main__":
    main()
