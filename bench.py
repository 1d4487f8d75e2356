#!/usr/bin/env python
"""Headline benchmark: mLSTM matmul-form forward + backward, B4 H8 S4096 D256 bf16 (fp32 accumulation), one MI355X.

One step = one forward (h, m, b) plus one backward (dq, dk, dv, df, di) through the C ABI of libmlstm_hip.so, inputs
resident in HBM.  Prints ONE JSON line.  `value` is algorithmic TFLOP/s: 7*D*S*(S+1) useful (causal) multiply-add
flops per head and step (2 products forward, 5 backward) divided by wall time; tokens/s is reported beside it.
`roofline` is the dominant kernel (the column-parallel backward tile kernel) timed with HIP events on its launch
stream during the timed steps; `cpu_baseline` times the C restatement of the reference's CPU path on one head.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

WORKLOADS = {
    # name: (B, NH, S, D, dtype, f_mean, i_mean, dh_std)
    "cfg4_B4_H8_S4096_D256_bf16": (4, 8, 4096, 256, torch.bfloat16, 3.0, 0.0, 1.0),
    "cfg5_B2_H32_S16384_D128_bf16": (2, 32, 16384, 128, torch.bfloat16, 3.0, -1.0, 0.1),
    "cfg2_B1_H4_S2048_D64_f32": (1, 4, 2048, 64, torch.float32, 0.0, 0.0, 1.0),
    "aux_B4_H16_S4096_D128_bf16": (4, 16, 4096, 128, torch.bfloat16, 3.0, 0.0, 1.0),
    "aux_B4_H8_S4096_D256_f16": (4, 8, 4096, 256, torch.float16, 3.0, 0.0, 1.0),
}
PEAK_TFLOPS = {torch.bfloat16: 2500.0, torch.float16: 2500.0, torch.float32: 157.3}
# HBM bytes per launch of the column kernel (in chunks of 512, the default at this shape), from two `rocprofv3 --pmc`
# runs of this script with --calibrate-copy (FETCH_SIZE 172673, WRITE_SIZE 142080 per dispatch; the 256 MiB copy in the
# same runs reads 131096 / 262144, so the fetch counter is scaled by 2.0 and the write counter by 1.0; both are then KiB).
COL_KERNEL_HBM_BYTES = {"cfg4_B4_H8_S4096_D256_bf16": (2.0 * 172673 + 1.0 * 142080) * 1024}
DTYPE_NAME = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}


def cpu_baseline(S, D, f_mean, heads=3):
    """`heads` of the workload's heads through the C oracle (dense S x S, fp32, single thread like the reference's
    cpu_utils.cuh): about 4.4 s per head at S=4096, D=256 on the GPU box's host.  Returns the JSON object."""
    import numpy as np
    from oracle import c_oracle as C
    dt = 0.0
    for head in range(heads):
        rng = np.random.default_rng(head)
        q, k, v, dh = (rng.standard_normal((S, D)).astype(np.float32) for _ in range(4))
        f = (rng.standard_normal(S) + f_mean).astype(np.float32)
        i = rng.standard_normal(S).astype(np.float32)
        t0 = time.perf_counter()
        C.forward_f32(q, k, v, f, i, threads=1)
        C.backward_f32(dh, q, k, v, f, i, threads=1)
        dt += time.perf_counter() - t0
    flops = heads * 7.0 * D * S * (S + 1)
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": f"{heads} of the workload's heads (S={S}, D={D}), forward+backward, oracle/mlstm_cpu.c, {dt:.1f} s",
            "tokens_per_s": heads * S / dt}


def bench_scan(args, ffi):
    """Secondary workload: scan form, B1 H4 S2048 D1024 fp32 (the reference's own scan self-check shape)."""
    L = ffi.lib()
    B, NH, S, D = 1, 4, 2048, 1024
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    mk = lambda *s: torch.randn(s, generator=g, device=dev, dtype=torch.float32)
    q, k, v, o = (mk(B, NH, S, D) for _ in range(4))
    f, i = mk(B, NH, S), mk(B, NH, S)
    h = torch.empty_like(q)
    ws, ws_n = ffi.workspace(ffi.OP_SCAN_FORWARD, B, NH, S, D, ffi.F32, dev)
    st, P = ffi.stream_ptr(), ffi.ptr

    def step():
        ffi.check_rc(L.mlstm_scan_forward_ex(P(q), P(k), P(v), P(f), P(i), P(o), P(h), B, NH, S, D, ffi.F32, P(ws), ws_n, st),
                     "mlstm_scan_forward_ex")

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ffi.timing_enable(True)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ffi.timing_enable(False)
    kern = {name: ffi.timing_read(name) for name in ("gates", "scan_carry", "scan_state", "scan_out")}
    ms_step = (t1 - t0) * 1e3 / args.steps
    BH = B * NH
    bytes_compulsory = (5.0 * BH * S * D + 3.0 * BH * S) * 4          # q, k, v, o in, h out, f, i in (+ m)
    flops = BH * (S / 64.0) * (2 * 64 * D * D * 2 + 2 * 2 * D * 64 * 65 / 2 * 2)  # state update + read-out, in-chunk pairs
    st_ms = kern["scan_state"][0] / max(kern["scan_state"][1], 1)
    out = {
        "metric": "mLSTM scan-form forward, compulsory HBM GB/s, cfg3_B1_H4_S2048_D1024_f32",
        "value": bytes_compulsory / (ms_step * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "cfg3_B1_H4_S2048_D1024_f32", "B": B, "NH": NH, "S": S, "D": D},
        "tokens_per_s": B * S / (ms_step * 1e-3), "fp32_tflops": flops / (ms_step * 1e-3) / 1e12,
        "kernel_ms": {n: (t / c if c else None) for n, (t, c) in kern.items()},
        "roofline": {"bound": "mfma", "kernel": "scan_intra_kernel + scan_state_kernel (fp32 MFMA)",
                     "achieved": flops / (st_ms * 1e-3) / 1e12 if st_ms else 0.0, "peak": 157.3, "unit": "TFLOP/s",
                     "frac": (flops / (st_ms * 1e-3) / 1e12 / 157.3) if st_ms else 0.0, "traffic": None},
        "hbm_frac_compulsory": bytes_compulsory / (ms_step * 1e-3) / 8e12,
    }
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="cfg4_B4_H8_S4096_D256_bf16", choices=sorted(WORKLOADS) + ["cfg3_scan"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--precise", action="store_true", help="split mode of the 16-bit kernels (MLSTM_PRECISE)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (torch) before the steps: under rocprofv3 --pmc its "
                         "FETCH_SIZE / WRITE_SIZE readings calibrate the counters' unit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (every box has one); --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)

    from _mlstm_pkg import submodule
    ffi = submodule("_ffi")
    if args.workload == "cfg3_scan":
        return bench_scan(args, ffi)
    L = ffi.lib()
    B, NH, S, D, dtype, f_mean, i_mean, dh_std = WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    mk = lambda *s: torch.randn(s, generator=g, device=dev, dtype=torch.float32)
    q, k, v = (mk(B, NH, S, D).to(dtype) for _ in range(3))
    f = (mk(B, NH, S) + f_mean).to(dtype)
    i = (mk(B, NH, S) + i_mean).to(dtype)
    dh = (mk(B, NH, S, D) * dh_std).to(dtype)
    h, dq, dk, dv = (torch.empty_like(q) for _ in range(4))
    m, b = (torch.empty((B, NH, S), device=dev, dtype=torch.float32) for _ in range(2))
    df, di = torch.empty_like(f), torch.empty_like(i)
    dt_code = ffi.dtype_code(dtype, args.precise)
    gate_code = ffi.dtype_code(dtype)
    ws, ws_n = ffi.workspace(ffi.OP_BACKWARD, B, NH, S, D, dt_code, dev)
    st = ffi.stream_ptr()
    P = ffi.ptr

    # what Triton_mLSTM.apply(...).backward(dh) runs: the forward keeps (h, m, b) and, for sequences that run in chunks,
    # the states at the chunk ends for its backward
    nsaved = int(L.mlstm_saved_state_bytes(B, NH, S, D, dt_code))
    saved = torch.empty(max(nsaved, 1), dtype=torch.uint8, device=dev)

    def step():
        rc = L.mlstm_forward_save_ex(P(q), P(k), P(v), P(f), P(i), P(h), P(m), P(b), P(saved), nsaved, B, NH, S, D, dt_code, gate_code,
                                     P(ws), ws_n, st)
        ffi.check_rc(rc, "mlstm_forward_save_ex")
        rc = L.mlstm_backward_saved_ex(P(dh), P(q), P(k), P(v), P(f), P(i), P(h), P(m), P(b), P(saved), nsaved, P(dq), P(dk), P(dv),
                                       P(df), P(di), B, NH, S, D, dt_code, gate_code, P(ws), ws_n, st)
        ffi.check_rc(rc, "mlstm_backward_saved_ex")

    if args.calibrate_copy:
        src = torch.ones(64 * 1024 * 1024, device=dev, dtype=torch.float32)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # HIP events inside the timed region bracket the dominant kernel only, on every fourth step: an event pair holds
    # the stream idle for about 10 us, and with all six kernel groups timed on every step that was 9 % of the step
    ffi.timing_select(["col"], every=4)
    ffi.timing_enable(True)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    kern = {"col": ffi.timing_read("col")}
    # the other kernels' durations, for the breakdown: a few more steps, outside the timed region, all kernels timed
    ffi.timing_select(None, every=1)
    for _ in range(max(args.steps // 4, 1)):
        step()
    torch.cuda.synchronize()
    ffi.timing_enable(False)
    for name in ("gates", "chunk_states", "row_fwd", "row_dq", "df"):
        kern[name] = ffi.timing_read(name)
    ffi.timing_read("col")
    kern = {name: kern[name] for name in ("gates", "chunk_states", "row_fwd", "col", "row_dq", "df")}

    ms_step = (t1 - t0) * 1e3 / args.steps
    BH = B * NH
    unit_flops = float(D) * S * (S + 1) * BH            # one causal product over the whole batch
    flops_step = 7.0 * unit_flops
    tflops = flops_step / (ms_step * 1e-3) / 1e12
    tokens_s = B * S / (ms_step * 1e-3)

    # dominant kernel: column-parallel backward tile kernel, 3 of the 7 algorithmic products (QK^T recompute, dK, dV);
    # the fourth product it executes (dH V^T) is counted once, in the dQ kernel's share.  In chunks it only meets the
    # (query, key) pairs inside a chunk and its algorithmic work is counted over those pairs, sum over the chunks of
    # D * len * (len + 1) per product and head, plus the two products keys x reverse state (2 D^2 per key and product)
    # that bring in the queries behind the chunk.
    col_ms = kern["col"][0] / max(kern["col"][1], 1)
    chunk = int(L.mlstm_chunk_length_for(S, D, dt_code))
    el = torch.empty(0, dtype=dtype).element_size()
    if chunk > 0 and (S + 63) // 64 <= 1024:
        lens = [min(chunk, S - c0) for c0 in range(0, S, chunk)]
        col_unit = float(D) * sum(n * (n + 1) for n in lens) * BH
        state_flops = 2.0 * 2.0 * D * D * sum(lens[:-1]) * BH
        state_bytes = (len(lens) - 1) * (2.0 * D * D * el + 4.0 * D)
    else:
        chunk, col_unit, state_flops, state_bytes = 0, unit_flops, 0.0, 0.0
    col_flops = 3.0 * col_unit + state_flops
    peak = PEAK_TFLOPS[dtype]
    achieved = col_flops / (col_ms * 1e-3) / 1e12 if col_ms > 0 else 0.0
    # its compulsory HBM bytes: Q, dH, K, V once; dK, dV written; the row partials of the key tiles a position meets;
    # in chunks the reverse states in both layouts and their vectors
    tiles_met = sum((min(chunk, S - c0) // 64 + 1) / 2.0 * min(chunk, S - c0) for c0 in range(0, S, chunk)) if chunk else (S / 64 + 1) / 2.0 * S
    col_bytes = BH * (S * D * el * 6 + tiles_met * 4 + state_bytes)
    hbm_achieved = col_bytes / (col_ms * 1e-3) / 1e9 if col_ms > 0 else 0.0
    out = {
        "metric": "mLSTM matmul-form fwd+bwd algorithmic TFLOP/s (7*D*S*(S+1) per head), " + args.workload,
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": DTYPE_NAME[dtype], "data": "synthetic",
        "config": {"workload": args.workload, "B": B, "NH": NH, "S": S, "D": D, "f": f"N({f_mean},1)", "i": f"N({i_mean},1)"},
        "tokens_per_s": tokens_s,
        "frac_of_peak": tflops / peak,
        "kernel_ms": {n: (t / c if c else None) for n, (t, c) in kern.items()},
    }
    traffic = COL_KERNEL_HBM_BYTES.get(args.workload) if chunk == 512 or not chunk else None
    if achieved / peak >= hbm_achieved / 8000.0:
        out["roofline"] = {"bound": "mfma", "kernel": "col16_kernel (dK, dV, dI)", "achieved": achieved, "peak": peak,
                           "unit": "TFLOP/s", "frac": achieved / peak, "traffic": traffic}
    else:
        # in chunks a workgroup meets few query tiles and the kernel is nearer to the HBM roof than to the MFMA roof
        out["roofline"] = {"bound": "hbm", "kernel": "col16_kernel (dK, dV, dI), chunks of %d" % chunk, "achieved": hbm_achieved,
                           "peak": 8000.0, "unit": "GB/s", "frac": hbm_achieved / 8000.0, "traffic": traffic,
                           "mfma_tflops": achieved, "mfma_frac": achieved / peak}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(S, D, f_mean)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
