#!/usr/bin/env python
"""Headline benchmark: mLSTM matmul-form forward + backward, B4 H8 S4096 D256 bf16 (fp32 accumulation), one MI355X.

One step = one forward (h, m, b) plus one backward (dq, dk, dv, df, di) through the C ABI of libmlstm_hip.so, inputs
resident in HBM (the same buffers every step: 256 MiB of them, which the chip's 256 MB last-level cache may keep).
Prints ONE JSON line.  `value` is TIME TO SOLUTION expressed in the parallel form's flops: 7*D*S*(S+1) useful (causal)
multiply-add flops per head and step (2 products forward, 5 backward) divided by wall time.  It is not a hardware rate: long
16-bit sequences run in chunks and execute far fewer flops than that, which `executed_tflops` / `executed_frac` (also inside
the roofline object) report beside it; `tokens_per_s` is the same time as a rate of positions.  `roofline` is the dominant kernel (the
column-parallel backward tile kernel) timed with HIP events on its launch stream during the timed steps;
`cpu_baseline` times the C restatement of the reference's CPU path, `cpu_baseline_torch` the dense PyTorch formulas, on
the same seeded inputs; `secondary` holds the other workloads (long context, scan form, split mode, sLSTM cell), each measured the
same way (the tile and scan workloads with a roofline object of their own).
"""
import argparse
import hashlib
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
    "aux_B4_H8_S4096_D64_bf16": (4, 8, 4096, 64, torch.bfloat16, 3.0, 0.0, 1.0),
    "aux_B2_H8_S4096_D128_f32": (2, 8, 4096, 128, torch.float32, 3.0, 0.0, 1.0),
    "aux_B4_H8_S4096_D64_f32": (4, 8, 4096, 64, torch.float32, 3.0, 0.0, 1.0),
}
COLUMN_KERNEL = 0   # --column-kernel
PEAK_TFLOPS = {torch.bfloat16: 2500.0, torch.float16: 2500.0, torch.float32: 157.3}
DTYPE_NAME = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}
CSRC = os.path.join(ROOT, "xlstm-triton-cuda-implementation_amd", "csrc")


def kernel_source_hash():
    """Identifies the kernels a measured traffic figure belongs to: sha256 over the device sources of the mLSTM kernels
    (mlstm_*.hip and the headers they share; the sLSTM cell is a file of its own that none of them includes)."""
    hsh = hashlib.sha256()
    for name in sorted(os.listdir(CSRC)):
        if name.startswith("mlstm_") and name.endswith((".hip", ".h")):
            hsh.update(name.encode())
            hsh.update(open(os.path.join(CSRC, name), "rb").read())
    return hsh.hexdigest()[:16]


def measured_traffic(workload, kernel, chunk):
    """HBM bytes per launch of `kernel` from profiles/traffic.json (two rocprofv3 --pmc runs, see the file), or None when the
    figure on file was taken with other kernel sources or another chunk length."""
    try:
        table = json.load(open(os.path.join(ROOT, "profiles", "traffic.json")))
    except (OSError, ValueError):
        return None
    rec = table.get(workload, {}).get(kernel)
    if not rec or rec.get("source_hash") != kernel_source_hash() or rec.get("chunk_len") != chunk:
        return None
    return float(rec["hbm_bytes_per_launch"])


def make_inputs(B, NH, S, D, dtype, f_mean, i_mean, dh_std, with_o=False, seed=0):
    """The seeded recipe shared by the tests, the CPU baselines and this benchmark: one CPU generator, fp32 normal draws in
    the order q, k, v, f, i, dh (, o), affine transform, cast to the workload's type."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((B, NH, S, D), generator=g)
    k = torch.randn((B, NH, S, D), generator=g)
    v = torch.randn((B, NH, S, D), generator=g)
    f = torch.randn((B, NH, S), generator=g) + f_mean
    i = torch.randn((B, NH, S), generator=g) + i_mean
    dh = torch.randn((B, NH, S, D), generator=g) * dh_std
    out = [q, k, v, f, i, dh]
    if with_o:
        out.append(torch.randn((B, NH, S, D), generator=g))
    return [x.to(dtype) for x in out]


def cpu_baseline(host, S, D, heads=3):
    """`heads` of the workload's heads (its own seeded inputs, upcast to fp32) through the C oracle: dense S x S, fp32,
    single thread like the reference's cpu_utils.cuh; about 4.4 s per head at S=4096, D=256 on the GPU box's host."""
    from oracle import c_oracle as C
    q, k, v, f, i, dh = host
    NH = q.shape[1]
    dt = 0.0
    for head in range(heads):
        bi, hi = divmod(head, NH)
        a = [x[bi, hi].float().numpy().copy() for x in (q, k, v, f, i, dh)]
        t0 = time.perf_counter()
        C.forward_f32(a[0], a[1], a[2], a[3], a[4], threads=1)
        C.backward_f32(a[5], a[0], a[1], a[2], a[3], a[4], threads=1)
        dt += time.perf_counter() - t0
    flops = heads * 7.0 * D * S * (S + 1)
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": f"{heads} of the workload's heads (S={S}, D={D}), forward+backward, oracle/mlstm_cpu.c, {dt:.1f} s",
            "tokens_per_s": heads * S / dt}


def cpu_baseline_torch(host, S, D, heads=2):
    """The dense PyTorch formulas of the reference (mlstm_matmul.py:104-118, :336-365, restated in oracle/mlstm_oracle.py)
    in fp32 on `heads` heads with torch's intra-op threads."""
    from oracle import mlstm_oracle as O
    q, k, v, f, i, dh = host
    NH = q.shape[1]
    dt = 0.0
    for head in range(heads):
        bi, hi = divmod(head, NH)
        a = [x[bi:bi + 1, hi:hi + 1] for x in (q, k, v, f, i, dh)]
        t0 = time.perf_counter()
        O.mlstm_forward_dense(*a[:5], dtype=torch.float32)
        O.mlstm_backward_dense(a[5], *a[:5], dtype=torch.float32)
        dt += time.perf_counter() - t0
    flops = heads * 7.0 * D * S * (S + 1)
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{heads} of the workload's heads (S={S}, D={D}), forward+backward, dense torch fp32 formulas, {dt:.1f} s",
            "tokens_per_s": heads * S / dt}


def chunk_work(S, D, BH, chunk, el, precise=False):
    """Flops the kernels execute per step in chunks of `chunk`, and the column kernel's share, with its compulsory bytes.
    ``precise``: split mode, every second product of a pair and every product with a state or a weighted row runs twice (on
    the hi and on the lo term), and the states are twice the bytes."""
    lens = [min(chunk, S - c0) for c0 in range(0, S, chunk)]
    pair_unit = float(D) * sum(n * (n + 1) for n in lens) * BH            # one product over the (query, key) pairs inside chunks
    state_rows = float(sum(lens[1:])) * BH                                 # positions that read a forward state
    state_keys = float(sum(lens[:-1])) * BH                                # positions that read a reverse state
    sums = 2.0 * D * D * (sum(lens[:-1]) + sum(lens[1:])) * BH             # chunk sums, both directions (2 D^2 per position)
    two = 2.0 if precise else 1.0
    executed = (12.0 if precise else 8.0) * pair_unit + two * (2.0 * D * D * 2 * state_rows + 2.0 * D * D * 2 * state_keys + sums)
    # four products per pair (six in split mode), two with the reverse state
    col_flops = (6.0 if precise else 4.0) * pair_unit + two * 2.0 * D * D * 2 * state_keys
    tiles_met = sum((n // 64 + 1) / 2.0 * n for n in lens)
    col_bytes = BH * (S * D * el * 6 + tiles_met * 4 + (len(lens) - 1) * (two * D * D * el + 4.0 * D))
    return executed, col_flops, col_bytes


def run_matmul(ffi, name, steps, warmup, precise=False, host=None):
    """Times `steps` forward + backward steps of one matmul-form workload.  Returns (json object, host inputs)."""
    L = ffi.lib()
    B, NH, S, D, dtype, f_mean, i_mean, dh_std = WORKLOADS[name]
    dev = torch.device("cuda:0")
    if host is None:
        host = make_inputs(B, NH, S, D, dtype, f_mean, i_mean, dh_std)
    q, k, v, f, i, dh = (x.to(dev) for x in host)
    h, dq, dk, dv = (torch.empty_like(q) for _ in range(4))
    m, b = (torch.empty((B, NH, S), device=dev, dtype=torch.float32) for _ in range(2))
    df, di = torch.empty_like(f), torch.empty_like(i)
    dt_code, gate_code = ffi.dtype_code(dtype, precise), ffi.dtype_code(dtype)
    ws, ws_n = ffi.workspace(ffi.OP_BACKWARD, B, NH, S, D, dt_code, dev)
    st, P = ffi.stream_ptr(), ffi.ptr
    # what Triton_mLSTM.apply(...).backward(dh) runs: the forward keeps (h, m, b) and what its backward can reuse
    nsaved = int(L.mlstm_saved_state_bytes(B, NH, S, D, dt_code))
    saved = torch.empty(max(nsaved, 1), dtype=torch.uint8, device=dev)

    def step():
        rc = L.mlstm_forward_save_ex(P(q), P(k), P(v), P(f), P(i), P(h), P(m), P(b), P(saved), nsaved, B, NH, S, D, dt_code, gate_code,
                                     P(ws), ws_n, st)
        ffi.check_rc(rc, "mlstm_forward_save_ex")
        rc = L.mlstm_backward_saved_ex(P(dh), P(q), P(k), P(v), P(f), P(i), P(h), P(m), P(b), P(saved), nsaved, P(dq), P(dk), P(dv),
                                       P(df), P(di), B, NH, S, D, dt_code, gate_code, P(ws), ws_n, st)
        ffi.check_rc(rc, "mlstm_backward_saved_ex")

    # The per-kernel breakdown comes first: steps of its own with every kernel bracketed by HIP events, outside the timed
    # region (a few unbracketed ones ahead of them, so that the first launches' one-time costs stay out of the averages).
    # At least 50, for steady averages; behind them the GPU's clock has settled as well, which a short run straight from
    # idle does not reach (the first tens of steps after idle run 5-10 % slower) -- `breakdown_steps` in the output says
    # how many ran.
    breakdown_steps = max(steps // 4, 50)
    for _ in range(3):
        step()
    torch.cuda.synchronize()
    ffi.timing_select(None, every=1)
    ffi.timing_enable(True)
    for _ in range(breakdown_steps):
        step()
    torch.cuda.synchronize()
    ffi.timing_enable(False)
    kern = {kname: ffi.timing_read(kname) for kname in ("gates", "chunk_states", "row_fwd", "row_dq", "df")}
    ffi.timing_read("col")
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # HIP events inside the timed region bracket the dominant kernel only, on every fourth step: an event pair holds
    # the stream idle for about 10 us, and with all six kernel groups timed on every step that was 9 % of the step
    ffi.timing_select(["col"], every=4)
    ffi.timing_enable(True)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ffi.timing_enable(False)
    kern["col"] = ffi.timing_read("col")
    ffi.timing_select(None, every=1)
    kern = {kname: kern[kname] for kname in ("gates", "chunk_states", "row_fwd", "col", "row_dq", "df")}
    assert L.mlstm_kernel_error() == 0, "a kernel's bounded wait expired during the benchmark"

    ms_step = (t1 - t0) * 1e3 / steps
    BH = B * NH
    unit_flops = float(D) * S * (S + 1) * BH            # one causal product over the whole batch
    tflops = 7.0 * unit_flops / (ms_step * 1e-3) / 1e12
    peak = PEAK_TFLOPS[dtype]
    col_ms = kern["col"][0] / max(kern["col"][1], 1)
    chunk = int(L.mlstm_chunk_length_for(S, D, dt_code))
    el = torch.empty(0, dtype=dtype).element_size()
    if chunk > 0 and (S + 63) // 64 <= 1024:
        executed, col_flops, col_bytes = chunk_work(S, D, BH, chunk, el, precise)
    else:
        # every key tile: 8 products executed (dH V^T in both backward kernels), 4 of them in the column kernel; the split
        # mode runs each of the 4 second products (P V, G K, G^T Q, W^T dH) a second time on the low-order terms
        chunk = 0
        executed = (12.0 if precise else 8.0) * unit_flops
        col_flops = (6.0 if precise else 4.0) * unit_flops
        col_bytes = BH * (S * D * el * 6 + (S / 64 + 1) / 2.0 * S * 4)
    achieved = col_flops / (col_ms * 1e-3) / 1e12 if col_ms > 0 else 0.0
    hbm_achieved = col_bytes / (col_ms * 1e-3) / 1e9 if col_ms > 0 else 0.0
    variant = {0: "cold_kernel", 1: "col16_kernel", 2: "cold_kernel", 3: "col_kernel"}[COLUMN_KERNEL]
    col_kernel = "col_kernel" if (dtype == torch.float32 or D == 64) else ("cold_kernel" if precise and variant == "col16_kernel" else variant)
    traffic = measured_traffic(name + ("+precise" if precise else ""), col_kernel, chunk)
    out = {
        "metric": "mLSTM matmul-form fwd+bwd, time to solution as parallel-form TFLOP/s (7*D*S*(S+1) flops per head; not a hardware "
                  "rate: see executed_tflops) and tokens/s, " + name + (" split mode" if precise else ""),
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "breakdown_steps": breakdown_steps,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": DTYPE_NAME[dtype], "data": "synthetic",
        "config": {"workload": name, "B": B, "NH": NH, "S": S, "D": D, "f": f"N({f_mean},1)", "i": f"N({i_mean},1)",
                   "chunk_len": chunk, "split_mode": bool(precise)},
        "tokens_per_s": B * S / (ms_step * 1e-3),
        "algorithmic_frac": tflops / peak,
        "executed_tflops": executed / (ms_step * 1e-3) / 1e12,
        "executed_frac": executed / (ms_step * 1e-3) / 1e12 / peak,
        "kernel_ms": {n: (t / c if c else None) for n, (t, c) in kern.items()},
    }
    # (the step's executed flops ride along in the roofline object: the headline value is not a hardware rate)
    mfma = {"mfma_tflops": achieved, "mfma_frac": achieved / peak, "executed_tflops": out["executed_tflops"], "executed_frac": out["executed_frac"]}
    hbm = {"hbm_gbs": hbm_achieved, "hbm_frac": hbm_achieved / 8000.0, "executed_tflops": out["executed_tflops"],
           "executed_frac": out["executed_frac"]}
    if achieved / peak >= hbm_achieved / 8000.0:
        out["roofline"] = {"bound": "mfma", "kernel": col_kernel + " (dK, dV, dI)", "achieved": achieved, "peak": peak,
                           "unit": "TFLOP/s", "frac": achieved / peak, "traffic": traffic, **hbm}
    else:
        # in chunks a workgroup meets few query tiles and the kernel is nearer to the HBM roof than to the MFMA roof
        out["roofline"] = {"bound": "hbm", "kernel": col_kernel + " (dK, dV, dI), chunks of %d" % chunk, "achieved": hbm_achieved,
                           "peak": 8000.0, "unit": "GB/s", "frac": hbm_achieved / 8000.0, "traffic": traffic, **mfma}
    return out, host


def run_scan(ffi, steps, warmup, backward=False, shape=(1, 4, 2048, 1024), tag="cfg3"):
    """Scan form, B1 H4 S2048 D1024 fp32 (the reference's own scan self-check shape) unless ``shape`` says otherwise;
    ``backward``: a step is the forward followed by the backward (which recomputes the forward: five passes of the state
    kernel in all)."""
    L = ffi.lib()
    B, NH, S, D = shape
    wl = "%s_B%d_H%d_S%d_D%d_f32" % (tag, B, NH, S, D)
    dev = torch.device("cuda:0")
    host = make_inputs(B, NH, S, D, torch.float32, 0.0, 0.0, 1.0, with_o=True)
    q, k, v, f, i, dh, o = (x.to(dev) for x in host)
    h = torch.empty_like(q)
    ws, ws_n = ffi.workspace(ffi.OP_SCAN_FORWARD, B, NH, S, D, ffi.F32, dev)
    st, P = ffi.stream_ptr(), ffi.ptr
    if backward:   # a training step: the forward keeps its ungated output and normaliser sums for the backward
        hu, bsum = torch.empty_like(q), torch.empty_like(f)
        dq, dk, dv, do = (torch.empty_like(q) for _ in range(4))
        df, di = torch.empty_like(f), torch.empty_like(i)
        wsb, wsb_n = ffi.workspace(ffi.OP_SCAN_BACKWARD, B, NH, S, D, ffi.F32, dev)

    def step():
        if backward:
            ffi.check_rc(L.mlstm_scan_forward_save_ex(P(q), P(k), P(v), P(f), P(i), P(o), P(h), P(hu), P(bsum), B, NH, S, D, ffi.F32,
                                                      P(ws), ws_n, st), "mlstm_scan_forward_save_ex")
            ffi.check_rc(L.mlstm_scan_backward_saved_ex(P(dh), P(q), P(k), P(v), P(f), P(i), P(o), P(hu), P(bsum), P(dq), P(dk), P(dv),
                                                        P(df), P(di), P(do), B, NH, S, D, ffi.F32, P(wsb), wsb_n, st),
                         "mlstm_scan_backward_saved_ex")
        else:
            ffi.check_rc(L.mlstm_scan_forward_ex(P(q), P(k), P(v), P(f), P(i), P(o), P(h), B, NH, S, D, ffi.F32, P(ws), ws_n, st),
                         "mlstm_scan_forward_ex")

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ffi.timing_select(None, every=1)
    ffi.timing_enable(True)
    for _ in range(max(steps // 4, 1)):
        step()
    torch.cuda.synchronize()
    ffi.timing_enable(False)
    names = ("gates", "scan_carry", "scan_state", "scan_out") + (("scan_glue", "df") if backward else ())
    kern = {name: ffi.timing_read(name) for name in names}
    ms_step = (t1 - t0) * 1e3 / steps
    BH = B * NH
    # forward: q, k, v, o in, h out, f, i in (+ m); the backward adds dh in and six gradients out, reads q, k, v, o, f, i again,
    # and the ungated output travels from the one to the other
    bytes_compulsory = (5.0 * BH * S * D + 3.0 * BH * S) * 4 + (backward * (12.0 * BH * S * D + 6.0 * BH * S) * 4)
    flops = BH * (S / 64.0) * (2 * 64 * D * D * 2 + 2 * 2 * D * 64 * 65 / 2 * 2)  # state update + read-out, in-chunk pairs
    st_ms = kern["scan_state"][0] / max(kern["scan_state"][1], 1)   # (average over the passes of a step)
    t_fl = flops / (st_ms * 1e-3) / 1e12 if st_ms else 0.0
    flops *= 4 if backward else 1   # (the forward's walk and three more with other operands)
    return {
        "metric": "mLSTM scan-form %s, compulsory HBM GB/s, %s" % ("forward+backward" if backward else "forward", wl),
        "value": bytes_compulsory / (ms_step * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": wl, "B": B, "NH": NH, "S": S, "D": D},
        "tokens_per_s": B * S / (ms_step * 1e-3), "fp32_tflops": flops / (ms_step * 1e-3) / 1e12,
        "kernel_ms": {n: (t / c if c else None) for n, (t, c) in kern.items()},
        # the binding roof: 38.7 GF of fp32 matrix work against 168 MB of compulsory traffic (ridge at 20 flop/B, the
        # workload has 230); both fractions are reported
        "roofline": {"bound": "mfma", "kernel": "scan_state_kernel (fp32 MFMA)", "achieved": t_fl, "peak": 157.3, "unit": "TFLOP/s",
                     "frac": t_fl / 157.3, "traffic": measured_traffic(wl, "scan_state_kernel", 64),
                     "hbm_gbs": bytes_compulsory / (ms_step * 1e-3) / 1e9, "hbm_frac": bytes_compulsory / (ms_step * 1e-3) / 8e12},
    }


def run_slstm(ffi, steps, warmup, shape=(16, 4, 2048, 64)):
    """sLSTM cell, forward (keeping the state for the backward) + backward, fp32.  The recurrence through h is sequential in
    t: one workgroup per (batch, head) walks the sequence, so what is measured is the time of one step of that walk."""
    L = ffi.lib()
    B, NH, S, DH = shape
    wl = f"slstm_B{B}_NH{NH}_S{S}_DH{DH}_f32"
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    wx = torch.randn((B, S, 4, NH, DH), generator=g).to(dev)
    r = (torch.randn((NH, 4, DH, DH), generator=g) * DH ** -0.5).to(dev)
    b = (torch.randn((NH, 4, DH), generator=g) * 0.1).to(dev)
    dh = torch.randn((B, S, NH, DH), generator=g).to(dev)
    h = torch.empty_like(dh)
    saved = torch.empty(int(L.slstm_saved_bytes(B, NH, S, DH)), dtype=torch.uint8, device=dev)
    ws_n = int(L.slstm_workspace_bytes(B, NH, S, DH))
    ws = torch.empty(ws_n, dtype=torch.uint8, device=dev)
    dwx, dr, db = torch.empty_like(wx), torch.empty_like(r), torch.empty_like(b)
    st, P = ffi.stream_ptr(), ffi.ptr

    def fwd():
        ffi.check_rc(L.slstm_forward_ex(P(wx), P(r), P(b), P(h), P(saved), B, NH, S, DH, 1, st), "slstm_forward_ex")

    def bwd():
        ffi.check_rc(L.slstm_backward_ex(P(dh), P(h), P(r), P(saved), P(dwx), P(dr), P(db), B, NH, S, DH, 1, P(ws), ws_n, st),
                     "slstm_backward_ex")

    for _ in range(warmup):
        fwd(); bwd()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fwd(); bwd()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]   # (the calls run on torch's current stream)
    f_ms = b_ms = 0.0
    for _ in range(max(steps // 4, 1)):
        ev[0].record(); fwd(); ev[1].record(); bwd(); ev[2].record()
        torch.cuda.synchronize()
        f_ms += ev[0].elapsed_time(ev[1]); b_ms += ev[1].elapsed_time(ev[2])
    f_ms /= max(steps // 4, 1); b_ms /= max(steps // 4, 1)
    ms_step = (t1 - t0) * 1e3 / steps
    # wx in, h and the seven kept values out; those and dh in, dwx out; dwx and h in again for dR and db
    bytes_compulsory = 29.0 * B * S * NH * DH * 4
    return {
        "metric": "sLSTM cell forward+backward, sequence positions per second, " + wl,
        "value": B * S / (ms_step * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic", "config": {"workload": wl, "B": B, "NH": NH, "S": S, "DH": DH, "forget": "sigmoid"},
        "forward_ms": f_ms, "backward_ms": b_ms,
        # the quantity the kernels are built around: wall time per step of the recurrence (B * NH walks side by side)
        "ns_per_recurrence_step": {"forward": f_ms * 1e6 / S, "backward": b_ms * 1e6 / S},
        # Latency model of the sequential walk: one wave per SIMD issues an instruction about every four cycles whatever it is,
        # the compiled step loops have 143 (forward) / 170 (backward) instructions, the clock under load is about 2.1 GHz:
        # the floor is instructions x 4 cycles per step; `frac` = that floor over the measured time per step.
        "roofline": {"bound": "latency", "kernel": "slstm_forward_kernel + slstm_backward_kernel (one step of the recurrence)",
                     "achieved": (f_ms + b_ms) * 1e6 / S, "peak": (143 + 170) * 4 / 2.1, "unit": "ns/step",
                     "frac": ((143 + 170) * 4 / 2.1) / ((f_ms + b_ms) * 1e6 / S) if f_ms + b_ms > 0 else None, "traffic": None},
        "hbm_gbs": bytes_compulsory / (ms_step * 1e-3) / 1e9, "hbm_frac": bytes_compulsory / (ms_step * 1e-3) / 8e12,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="cfg4_B4_H8_S4096_D256_bf16", choices=sorted(WORKLOADS) + ["cfg3_scan", "cfg3_scan_backward", "long_scan", "slstm"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true", help="skip the secondary workloads (long context, scan, split mode)")
    ap.add_argument("--precise", action="store_true", help="split mode of the 16-bit kernels (MLSTM_PRECISE)")
    ap.add_argument("--chunk-length", type=int, default=0,
                    help="measurement aid: chunk length of the 16-bit kernels (a multiple of 128; 0 = the library's choice, < 0 = no chunks)")
    ap.add_argument("--state-kernel", type=int, default=0, choices=[0, 1, 2],
                    help="measurement aid: 0 = the library's choice, 1 = chunk sums + carry, 2 = the one-pass kernel")
    ap.add_argument("--column-kernel", type=int, default=0, choices=[0, 1, 2, 3],
                    help="measurement aid: 0 = the library's choice, 1 = col16_kernel, 2 = cold_kernel, 3 = col_kernel")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (torch), twice, before the steps: under rocprofv3 --pmc its "
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
    global COLUMN_KERNEL
    COLUMN_KERNEL = args.column_kernel
    ffi.set_column_kernel(args.column_kernel)
    ffi.set_chunk_length(args.chunk_length)
    ffi.set_state_kernel(args.state_kernel)
    if args.calibrate_copy:
        # 1 GiB, copied twice: four times the chip's 256 MB last-level cache, so the second copy's source comes from HBM
        # (a source that still sits in that cache reads as almost no FETCH_SIZE at all)
        src = torch.ones(256 * 1024 * 1024, device="cuda:0", dtype=torch.float32)
        dst = torch.empty_like(src)
        dst.copy_(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.workload == "long_scan":   # one long sequence: the state walk runs in segments side by side
        print(json.dumps(run_scan(ffi, args.steps, args.warmup, shape=(1, 1, 65536, 128), tag="long")))
        return
    if args.workload == "slstm":
        print(json.dumps(run_slstm(ffi, args.steps, args.warmup)))
        return
    if args.workload in ("cfg3_scan", "cfg3_scan_backward"):
        print(json.dumps(run_scan(ffi, args.steps, args.warmup, backward=args.workload.endswith("backward"))))
        return
    out, host = run_matmul(ffi, args.workload, args.steps, args.warmup, precise=args.precise)
    headline = args.workload == "cfg4_B4_H8_S4096_D256_bf16" and not args.precise
    if headline and not args.no_secondary:
        few = max(min(args.steps, 20), 5)
        split = run_matmul(ffi, args.workload, few, 3, precise=True, host=host)[0]
        # the same workload on the path that meets rtol 2e-2 / atol 2e-3 on every element (MLSTM_PRECISE), beside the default
        # path's figures above, whose parity bound carries a rounding-noise term
        out["literal_tolerance_mode"] = {"ms_per_step": split["ms_per_step"], "value": split["value"], "unit": "TFLOP/s",
                                         "tokens_per_s": split["tokens_per_s"], "algorithmic_frac": split["algorithmic_frac"],
                                         "executed_frac": split["executed_frac"]}
        out["secondary"] = [split,
                            run_matmul(ffi, "cfg5_B2_H32_S16384_D128_bf16", few, 3)[0],
                            run_matmul(ffi, "cfg2_B1_H4_S2048_D64_f32", max(args.steps // 4, 10), 3)[0],
                            run_scan(ffi, max(args.steps, 20), 5), run_scan(ffi, max(args.steps // 4, 10), 3, backward=True),
                            run_slstm(ffi, max(args.steps // 4, 10), 3)]
    if not args.no_cpu_baseline:
        S, D = WORKLOADS[args.workload][2:4]
        out["cpu_baseline"] = cpu_baseline(host, S, D)
        out["cpu_baseline_torch"] = cpu_baseline_torch(host, S, D)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
