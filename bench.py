"""Headline benchmark: Wavefunction Embedding forward at B=1, N=16384, d_model=512
(BASELINE.json configs[1]) on one MI355X, with the geometric attention forward at
N=16384, H=8, d=64 measured beside it, roofline fractions for both kernels and
the CPU PyTorch path timed on the host cores as a baseline.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-attn]

Prints ONE JSON line.  A "step" is one WE forward over the whole batch, inputs
and outputs resident in HBM, outputs pre-allocated.
"""
import argparse
import json
import os
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

# HBM traffic per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (profiles/), bytes
# WE: FETCH_SIZE 4370.5 KiB x 2.0 (calibration factor of that counter) + WRITE_SIZE 82271.9 KiB x 1.0
WE_TRAFFIC_BYTES = int((4370.5 * 2.0 + 82271.9) * 1024)
# attention: FETCH_SIZE 43028.5 KiB x 2.0 (both distance-path bodies of the one launch) + WRITE_SIZE 33792.0 KiB x 1.0
ATTN_TRAFFIC_BYTES = int((43028.5 * 2.0 + 33792.0) * 1024)


def median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2]


def settle(torch, fn, min_ms=60.0):
    """Run fn untimed for at least min_ms: while a leg's inputs are made on the host the GPU idles and drops its
    clocks, and the first ~25 ms of work afterwards run below the sustained rate."""
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < min_ms:
        fn()
        torch.cuda.synchronize()


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-attn", action="store_true", help="skip the geometric attention leg")
    ap.add_argument("--no-aniso", action="store_true", help="skip the anisotropic WE leg")
    ap.add_argument("--no-encoder", action="store_true", help="skip the encoder-forward leg (BASELINE.json configs[3])")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target duration of the CPU baseline sample")
    ap.add_argument("--we-tuning", type=int, default=0)
    ap.add_argument("--copy-calib", action="store_true",
                    help="also launch a 256 MiB device copy, so a rocprofv3 --pmc run of this command holds a kernel of known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (observer rows and (batch, head) pairs are "
              "independent, so the work shards without any exchange); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from proteusai_amd import _lib, synth
    lib = _lib.load()
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    # ---------------- WE forward, B=1, N=16384, d_model=512, compacted random-walk chain ----------------
    Z, N, d_model = 1, 16384, 512
    coords, wn = synth.we_inputs(N, seed=2, batch=Z, d_model=d_model, compact=True)
    K = wn.numel()
    c, w = coords.to(dev).contiguous(), wn.to(dev)
    out = torch.empty(Z, N, 2 * K, device=dev)
    cs = torch.empty(Z, N, K, device=dev)
    ss = torch.empty(Z, N, K, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def we_step():
        rc = lib.proteus_we_fwd(c.data_ptr(), _lib.COORDS_AOS, w.data_ptr(), None, out.data_ptr(), cs.data_ptr(),
                                ss.data_ptr(), Z, N, K, args.we_tuning, stream)
        if rc != 0:
            _lib.check(rc, "proteus_we_fwd")

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

    rates = probe_rates(lib, torch, dev)
    # per unit: the phase product (scalar operand), v_sin, v_cos, two v_fmac and two v_add on vector operands
    r_trans = (rates["sin"] + rates["cos"]) / 2
    t_model_ms = W * (1.0 / rates["mul_s"] + 2.0 / rates["fmac_v"] + 2.0 / rates["add_v"] + 2.0 / r_trans) * 1e3
    achieved_tflops = 9.0 * W / (avg_kernel_ms * 1e-3) / 1e12   # 9 flop per unit, FMA counted as 2
    roofline = {
        "kernel": "we_fwd_kernel", "bound": "valu", "achieved": achieved_tflops, "peak": PEAK_FP32_VECTOR_TFLOPS,
        "unit": "TFLOP/s", "frac": achieved_tflops / PEAK_FP32_VECTOR_TFLOPS, "traffic": WE_TRAFFIC_BYTES,
        "kernel_ms": avg_kernel_ms,
        "issue_model": {
            "lane_ops_per_unit": {"mul_scalar_operand": 1, "fmac_vector_operands": 2, "add_vector_operands": 2,
                                  "transcendental": 2},
            "measured_lane_ops_per_s": {"mul_scalar_operand": rates["mul_s"], "fmac_vector_operands": rates["fmac_v"],
                                        "add_vector_operands": rates["add_v"], "transcendental": r_trans},
            "model_ms": t_model_ms, "frac": t_model_ms / avg_kernel_ms,
        },
    }

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

    # ---------------- the same forward without the cos/sin sums (inference: nothing kept for a backward) ----------
    def we_lean_step():
        rc = lib.proteus_we_fwd(c.data_ptr(), _lib.COORDS_AOS, w.data_ptr(), None, out.data_ptr(), None, None,
                                Z, N, K, args.we_tuning, stream)
        if rc != 0:
            _lib.check(rc, "proteus_we_fwd")
    for _ in range(2):
        we_lean_step()
    torch.cuda.synchronize()
    n_lean = max(5, args.steps // 2)
    lev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_lean)]
    for e0, e1 in lev:
        e0.record()
        we_lean_step()
        e1.record()
    torch.cuda.synchronize()
    lean_ms = sum(e0.elapsed_time(e1) for e0, e1 in lev) / n_lean
    # per unit: the phase product, v_sin, v_cos and two v_fmac (the two v_add of the plain sums are gone)
    lean_model_ms = W * (1.0 / rates["mul_s"] + 2.0 / rates["fmac_v"] + 2.0 / r_trans) * 1e3
    result["we_fwd_without_sums"] = {
        "workload": "the headline shape with cos_sums = sin_sums = NULL (embedding only; not the headline metric, "
                    "whose forward also returns the sums as the reference's does)",
        "ms": lean_ms, "gpair_wavenumber_per_s": W / (lean_ms * 1e-3) / 1e9, "dtype": "f32",
        "issue_model": {"model_ms": lean_model_ms, "frac": lean_model_ms / lean_ms},
    }

    # ---------------- WE backward (the reduction of dO against the sums), same shape: HBM-bound ----------------
    dO = torch.randn(Z, N, 2 * K, device=dev)
    dk = torch.empty(K, device=dev)
    ws_bytes = lib.proteus_we_bwd_workspace_bytes(Z, N, K)
    ws = torch.empty(ws_bytes // 4, device=dev)

    def we_bwd_step():
        rc = lib.proteus_we_bwd(dO.data_ptr(), cs.data_ptr(), ss.data_ptr(), dk.data_ptr(), ws.data_ptr(), ws_bytes,
                                Z, N, K, stream)
        if rc != 0:
            _lib.check(rc, "proteus_we_bwd")
    settle(torch, we_bwd_step)
    bev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(20)]
    for e0, e1 in bev:
        e0.record()
        we_bwd_step()
        e1.record()
    torch.cuda.synchronize()
    b_ms = sorted(e0.elapsed_time(e1) for e0, e1 in bev)[len(bev) // 2]
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
    if not args.no_aniso:
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
        for _ in range(2):
            aniso_step()
        torch.cuda.synchronize()
        n_it = max(5, args.steps // 2)
        xev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_it)]
        for e0, e1 in xev:
            e0.record()
            aniso_step()
            e1.record()
        torch.cuda.synchronize()
        x_ms = sum(e0.elapsed_time(e1) for e0, e1 in xev) / n_it
        # per unit: 2 scalar-operand phase ops, v_fract, 4 v_fmac + 2 v_add on vector operands, v_sin, v_cos
        x_model_ms = W * (2.0 / rates["mul_s"] + 1.0 / rates["fract"] + 4.0 / rates["fmac_v"] + 2.0 / rates["add_v"]
                          + 2.0 / r_trans) * 1e3
        result["we_aniso"] = {
            "workload": "anisotropic (C-beta scaled) WE forward, out + d_cb + d_k, B=1 N=16384 256 wavenumbers, same chain, random unit C-beta vectors",
            "ms": x_ms, "gpair_wavenumber_per_s": W / (x_ms * 1e-3) / 1e9, "dtype": "f32",
            "issue_model": {"lane_ops_per_unit": {"scalar_operand": 2, "fract": 1, "fmac_vector_operands": 4,
                                                  "add_vector_operands": 2, "transcendental": 2},
                            "model_ms": x_model_ms, "frac": x_model_ms / x_ms},
        }

    # ---------------- geometric attention forward, N=16384, H=8, d=64 (configs[4]) ----------------
    if not args.no_attn:
        wc, _ = synth.we_inputs(65536, seed=5, compact=True)
        Q, Kt, V, ac, sigma, _ = synth.attn_inputs(1, 8, 16384, 64, seed=5, coords=wc[:, :16384].contiguous())
        q, k, v, acd, sg = Q.to(dev), Kt.to(dev), V.to(dev), ac.to(dev), sigma.to(dev)
        O = torch.empty(1, 8, 16384, 64, device=dev)
        L = torch.empty(1, 8, 16384, device=dev)

        def attn_step():
            rc = lib.proteus_geo_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), acd.data_ptr(), sg.data_ptr(), None,
                                          O.data_ptr(), L.data_ptr(), 1, 8, 16384, 64, 0, stream)
            if rc != 0:
                _lib.check(rc, "proteus_geo_attn_fwd")
        settle(torch, attn_step)
        n_it = max(10, args.steps)
        aev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_it)]
        for e0, e1 in aev:
            e0.record()
            attn_step()
            e1.record()
        torch.cuda.synchronize()
        a_ms = sum(e0.elapsed_time(e1) for e0, e1 in aev) / n_it
        flops = 4.0 * 8 * 64 * 16384 * 16384
        a_tflops = flops / (a_ms * 1e-3) / 1e12
        result["geo_attn"] = {
            "workload": "geometric attention forward Z=1 H=8 N=16384 d_head=64 bf16, compacted chain, sigma 3-25 A (BASELINE.json configs[4])",
            "ms": a_ms, "tflops": a_tflops, "dtype": "bf16",
            "roofline": {"kernel": "geo_attn_fwd_kernel", "bound": "mfma", "achieved": a_tflops, "peak": PEAK_BF16_MFMA_TFLOPS,
                         "unit": "TFLOP/s", "frac": a_tflops / PEAK_BF16_MFMA_TFLOPS, "traffic": ATTN_TRAFFIC_BYTES},
        }

        # ---- backward of the same shape (dQ, dK, dV, d sigma from the forward's O and L) ----
        gq = torch.Generator().manual_seed(5)
        dOb = (torch.randn(1, 8, 16384, 64, generator=gq) / 8).bfloat16().to(dev)
        Dv = (O * dOb.float()).sum(-1).contiguous()
        dQ_, dK_, dV_ = (torch.empty(1, 8, 16384, 64, device=dev) for _ in range(3))
        dsg = torch.zeros(8, device=dev)

        def bwd_step():
            rc = lib.proteus_geo_attn_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), dOb.data_ptr(), acd.data_ptr(), sg.data_ptr(),
                                          None, None, L.data_ptr(), Dv.data_ptr(), dQ_.data_ptr(), dK_.data_ptr(), dV_.data_ptr(),
                                          dsg.data_ptr(), None, 1, 8, 16384, 64, 0.0, 1.0, stream)
            if rc != 0:
                _lib.check(rc, "proteus_geo_attn_bwd")
        settle(torch, bwd_step)
        bev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(5)]
        for e0, e1 in bev:
            e0.record()
            bwd_step()
            e1.record()
        torch.cuda.synchronize()
        b_ms = sum(e0.elapsed_time(e1) for e0, e1 in bev) / len(bev)
        result["geo_attn_bwd"] = {
            "workload": "geometric attention backward, same shape: dQ, dK, dV, d_sigma (two passes in one launch, S and dP recomputed in each)",
            "ms": b_ms, "tflops_5_products": 10.0 * 8 * 64 * 16384 * 16384 / (b_ms * 1e-3) / 1e12,
            "tflops_issued_7_products": 14.0 * 8 * 64 * 16384 * 16384 / (b_ms * 1e-3) / 1e12, "dtype": "bf16",
        }

    # ---------------- encoder forward, B=8, N=1024, 4 layers, bf16 weights, fp32 WE (configs[3]) ----------------
    if not args.no_encoder:
        import proteusai_amd as pa
        torch.manual_seed(4)
        model = pa.ProteusEncoder().eval().to(dev)
        model.aa_embedding.to(torch.bfloat16)
        model.layers.to(torch.bfloat16)
        model.head.to(torch.bfloat16)
        g = torch.Generator().manual_seed(4)
        ecoords = torch.stack([synth.random_walk_chain(1024, g) for _ in range(8)]).to(dev)
        etokens = torch.randint(0, 33, (8, 1024), generator=g).to(dev)
        lens = torch.randint(128, 1025, (8,), generator=g)
        emask = (torch.arange(1024)[None, :] >= lens[:, None]).to(dev)
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
        }
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

    # ---------------- CPU baseline: the tiled CPU PyTorch path on a bounded sample of observer rows ----------------
    if not args.no_cpu:
        from oracle import torch_oracle
        threads = torch.get_num_threads()
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
