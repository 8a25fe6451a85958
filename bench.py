#!/usr/bin/env python3
"""Benchmark of the compact RNN-T loss + gradient hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--no-cpu]

A step is one forward + backward of `cwarp_rnnt.transducer_loss(..., fused_log_softmax=True)` on
one synthetic batch that is already resident in HBM.  Prints ONE JSON line.

  value      algorithmic HBM bytes per step / wall time per step, in GB/s, where
             algorithmic bytes = R*V*(2*s_x + s_g): read the logits in the forward pass, read
             them again in the backward pass, write the gradient (R = sum T_i*(U_i+1)).
  roofline   the gradient kernel (the dominant one: 2/3 of the bytes) timed on its own with
             HIP events on the stream it is launched on, against the 8 TB/s HBM peak.
  cpu_baseline  the C restatement of the float64 oracle (OpenMP, all host cores of the process)
             timed on whole passes over the same batch for a bounded time; its outputs double as
             the parity check of the run.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16 matrix-core peak of MI355X
WORKLOADS = {
    1: "c1 tiny: N=4 T~U[8,32] U~U[2,10] V=32 fp32",
    2: "c2 BPE ASR: N=32 T~U[100,250] U~U[20,80] V=1024 fp32 logits N(0,2), blank=0, mean reduction",
    3: "c3 large vocab: N=16 T~U[150,300] U~U[40,120] V=4096 fp16 logits N(0,1)",
    4: "c4 ragged: N=64 T~logN(120,0.6) U~logN(30,0.7) incl. U=0 and T=1, V=512 fp32",
    5: "c5 long-form chars: N=4 T~U[1000,1500] U~U[200,400] V=128 fp32 logits N(0,1.5)",
}


def measured_traffic(kernel: str, config: int):
    """(HBM bytes per launch of `kernel`, file it was read from) from the committed rocprofv3 counter
    summary of this configuration, or (None, None)."""
    rel = os.path.join("profiles", f"traffic_c{config}.json.txt")
    try:
        with open(os.path.join(ROOT, rel)) as f:
            val = json.load(f).get(kernel)
        return val, (rel if val is not None else None)
    except (OSError, ValueError):
        return None, None


def cpu_baseline(cfg, x_cpu, budget_s, dev_out):
    """Time the C restatement of the oracle (oracle/rnnt_oracle_c.c: float64 arithmetic, OpenMP over
    the sequences of the batch, every host core the process may use) on whole passes over the same
    batch, for about the budget; the first pass's outputs double as the parity check of the device
    results (the C restatement is itself pinned to the NumPy oracle in tests/test_oracle_pins.py)."""
    import torch
    from oracle import build_c
    lib = build_c.load()
    x32 = x_cpu.to(dtype=torch.float32).numpy()
    N, V = cfg["N"], cfg["V"]
    esize = x_cpu.element_size()
    go = np.full(N, 1.0 / N)
    t_used, passes = 0.0, 0
    loss_rel = grad_abs = 0.0
    while True:
        t0 = time.perf_counter()
        ref = build_c.loss_and_grad(lib, x32, cfg["lx"], cfg["y_padded"], cfg["ly"], 0, True, go, want_G=False)
        dt = time.perf_counter() - t0
        t_used += dt
        passes += 1
        if passes == 1:
            loss_rel = float(np.max(np.abs(dev_out["costs"] - ref["costs"]) / np.abs(ref["costs"])))
            step = 1 << 16
            for a in range(0, x32.shape[0], step):
                grad_abs = max(grad_abs, float(np.abs(dev_out["grad"](a, a + step) - ref["grad"][a:a + step]).max()))
        del ref
        if t_used + dt > budget_s:
            break
    bytes_done = passes * x32.shape[0] * V * 3 * esize
    cores = int(lib.rnnt_oracle_c_threads())
    return dict(value=bytes_done / t_used / 1e9, unit="GB/s", cores=cores, kind="port",
                sample=f"C restatement of the float64 oracle (OpenMP over sequences, {cores} threads of "
                       f"{os.cpu_count()} host cpus), {passes} whole passes over the same batch, {t_used:.1f} s",
                ), dict(loss_rel_err=loss_rel, grad_abs_err=grad_abs, sequences_checked=N)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=30,
                    help="untimed steps; the first ~20 steps after an idle GPU run up to 15 % slower")
    ap.add_argument("--config", type=int, default=2, choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / parity leg")
    ap.add_argument("--cpu-budget", type=float, default=20.0, help="seconds of CPU work for the baseline")
    ap.add_argument("--with-pack", action="store_true",
                    help="also time the padded -> compact pack op and its backward on the padded form of the same "
                         "batch (reported under 'pack_op'; not part of 'value')")
    ap.add_argument("--with-fused-joiner", action="store_true",
                    help="also time the output layer fused into the loss (cwr_joint_forward / cwr_joint_backward) "
                         "against the route through stored logits")
    ap.add_argument("--joint-dim", type=int, default=512, help="H of --with-fused-joiner")
    ap.add_argument("--with-joiner", action="store_true",
                    help="also time the compact joiner front (broadcast sum + tanh for valid cells, H=512, in the "
                         "batch's storage type) and its backward at the same lengths (reported under 'joiner_op'; "
                         "not part of 'value')")
    ap.add_argument("--with-long-labels", action="store_true",
                    help="also time the forward call and its lattice stage on N=4, T=1250 and U = 300 ... 2300 labels "
                         "(log-prob mode, V=4: the lattice dominates; reported under 'long_labels')")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (known traffic) so that a counter run can scale "
                         "FETCH_SIZE / WRITE_SIZE against it")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path is measured on ONE GPU (every sequence is independent, so a "
                 "data-parallel trainer gives each GPU its own batch); run with --gpus 1")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    import compactwarprnntloss_amd as pkg
    import cwarp_rnnt
    from compactwarprnntloss_amd import workloads

    dev = torch.device("cuda:0")
    cfg = workloads.make_config(args.config)
    tdt = torch.float16 if cfg["dtype"] == "f16" else torch.float32
    g = torch.Generator(device="cpu").manual_seed(1000 + args.config)
    # generated on the host in fp32, rounded once to the storage type, then made resident
    x_cpu = (torch.randn((cfg["R"], cfg["V"]), generator=g, dtype=torch.float32) * cfg["sigma"]).to(tdt)
    x = x_cpu.to(dev).requires_grad_(True)
    lx = torch.from_numpy(cfg["lx"]).to(dev)
    ly = torch.from_numpy(cfg["ly"]).to(dev)
    y = torch.from_numpy(cfg["y_padded"]).to(dev)
    R, V, N = cfg["R"], cfg["V"], cfg["N"]
    esize = x.element_size()
    bytes_step = R * V * 3 * esize

    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    def step():
        x.grad = None
        loss = cwarp_rnnt.transducer_loss(x, lx, y, ly, 0, "mean", gather=True, fused_log_softmax=True)
        loss.backward()
        return loss

    # After any idle period (0.2 s is enough) this GPU runs the first ~12 ms of streaming work up to
    # 15 % slower, whatever the kernels are.  Two priming steps let the allocator fetch its blocks
    # (the device idles meanwhile), then ~25 ms of plain device copies, queued without a gap in
    # front of the warm-up steps, bring the GPU to its steady state, so that a short --warmup does
    # not measure that transient.
    src = torch.empty(1 << 27, dtype=torch.float32, device=dev)
    dst = torch.empty_like(src)
    for _ in range(2):
        step()
    torch.cuda.synchronize()
    for _ in range(120):
        dst.copy_(src)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    del src, dst
    # events between the steps (recorded, never waited on inside the timed region) give the spread
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for k in range(args.steps):
        step()
        marks[k + 1].record()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps
    per_step = sorted(marks[k].elapsed_time(marks[k + 1]) for k in range(args.steps))

    # per-call timing with events on the stream the kernels run on (torch's current stream)
    xd = x.detach()
    costs, st = pkg.rnnt_forward(xd, lx, y, ly, 0, True)
    go = torch.full((N,), 1.0 / N, device=dev)
    out = torch.empty_like(xd)
    iters = max(10, args.steps)

    def timed(fn):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        e1.synchronize()
        return e0.elapsed_time(e1) / iters

    bwd_ms = timed(lambda: pkg.rnnt_backward(xd, lx, y, ly, 0, st, go, out=out))
    fwd_ms = timed(lambda: pkg.rnnt_forward(xd, lx, y, ly, 0, True))
    nograd_ms = timed(lambda: pkg.rnnt_forward(xd, lx, y, ly, 0, True, with_grad=False))

    # Latency breakdown of the forward call: HIP events between its four stages (a measurement hook of
    # the library; each figure holds the kernel and the dependency gap in front of it), the gradient
    # pass from the backward call above.  One anti-diagonal = one frame or label of the sequence with
    # the most of them; the lattice walk is a serial chain over those.
    import ctypes as C
    lib = pkg._lib.load()
    stage = (C.c_float * 4)()
    lat_runs = []
    for _ in range(max(10, args.steps // 2)):
        rc = lib.cwr_debug_forward_stage_times(
            xd.data_ptr(), pkg.loss._DTYPES[xd.dtype], R, V, lx.data_ptr(), ly.data_ptr(), y.data_ptr(), y.size(1),
            y.numel(), N, 0, pkg._lib.MODE_FUSED, st.max_u, st.workspace.data_ptr(), st.workspace.numel(),
            st.row_off.data_ptr(), st.lab_off.data_ptr(), st.status.data_ptr(), st.rowinfo.data_ptr(),
            st.lse.data_ptr(), st.grads.data_ptr(), costs.data_ptr(), torch.cuda.current_stream().cuda_stream, stage)
        if rc != 0:
            sys.exit("cwr_debug_forward_stage_times: " + pkg._lib.strerror(rc))
        lat_runs.append(list(stage))
    lat = [sorted(r[i] for r in lat_runs)[len(lat_runs) // 2] for i in range(4)]  # medians
    diagonals = int((cfg["lx"].astype(np.int64) + cfg["ly"]).max())
    # the walk serves two label positions per lane and step: T + ceil((U+1)/2) - 1 steps per sequence
    walk_steps = int((cfg["lx"].astype(np.int64) + (cfg["ly"].astype(np.int64) + 2) // 2 - 1).max())

    grad_bytes = R * V * 2 * esize
    achieved = grad_bytes / (bwd_ms * 1e-3) / 1e9
    traffic, traffic_source = measured_traffic("k_grad", args.config)
    result = {
        "metric": "fwd+bwd algorithmic HBM GB/s of the fused compact RNN-T loss (gather+loss+grad)",
        "value": round(bytes_step / (ms_step * 1e-3) / 1e9, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16" if cfg["dtype"] == "f16" else "f32",
        "data": "synthetic",
        "config": {"workload": WORKLOADS[args.config], "N": N, "R": R, "V": V,
                   "algorithmic_bytes_per_step": bytes_step, "entry": "cwarp_rnnt.transducer_loss"},
        "pct_of_hbm_peak": round(100.0 * bytes_step / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
        "step_ms": {"median": round(per_step[len(per_step) // 2], 4), "min": round(per_step[0], 4),
                    "max": round(per_step[-1], 4)},
        "breakdown_ms": {"forward_call": round(fwd_ms, 4), "backward_call": round(bwd_ms, 4),
                         "forward_nograd_call": round(nograd_ms, 4)},
        "latency_us": {"offsets": round(lat[0], 2), "gather": round(lat[1], 2), "lattice": round(lat[2], 2),
                       "fill": round(lat[3], 2), "grad": round(bwd_ms * 1e3, 2),
                       "lattice_ns_per_diagonal": round(lat[2] * 1e3 / diagonals, 1),
                       "diagonals_longest_sequence": diagonals,
                       "lattice_ns_per_walk_step": round(lat[2] * 1e3 / walk_steps, 1),
                       "walk_steps_longest_sequence": walk_steps,
                       "how": "medians of HIP-event intervals between the stages of one forward call "
                              "(cwr_debug_forward_stage_times); grad = the backward call"},
        "roofline": {"bound": "hbm", "kernel": "k_grad (cwr_backward)", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": traffic, "traffic_source": traffic_source},
    }

    if args.with_long_labels:
        # Label sequences beyond one workgroup's concurrent strips: up to 1023 labels a sequence is walked
        # by one wave per strip of 128 labels at once; from 1024 on one wave walks the strips in turn.
        import ctypes as C
        lib = pkg._lib.load()
        rows = []
        for U in (300, 511, 600, 1000, 1023, 1200, 2000, 2300):
            Nl, Tl, Vl = 4, 1250, 4
            lxl = torch.full((Nl,), Tl, dtype=torch.int32, device=dev)
            lyl = torch.full((Nl,), U, dtype=torch.int32, device=dev)
            Rl = Nl * Tl * (U + 1)
            xl = torch.log_softmax(torch.randn((Rl, Vl), device=dev), dim=1)
            yl = torch.randint(1, Vl, (Nl, U), dtype=torch.int32, device=dev)
            cl, stl = pkg.rnnt_forward(xl, lxl, yl, lyl, 0, False)
            stage = (C.c_float * 4)()
            runs = []
            for _ in range(7):
                rc = lib.cwr_debug_forward_stage_times(
                    xl.data_ptr(), pkg.loss._DTYPES[xl.dtype], Rl, Vl, lxl.data_ptr(), lyl.data_ptr(), yl.data_ptr(), U,
                    yl.numel(), Nl, 0, pkg._lib.MODE_LOGPROB, stl.max_u, stl.workspace.data_ptr(),
                    stl.workspace.numel(), stl.row_off.data_ptr(), stl.lab_off.data_ptr(), stl.status.data_ptr(),
                    stl.rowinfo.data_ptr(), None, stl.grads.data_ptr(), cl.data_ptr(),
                    torch.cuda.current_stream().cuda_stream, stage)
                if rc != 0:
                    sys.exit("cwr_debug_forward_stage_times: " + pkg._lib.strerror(rc))
                runs.append(list(stage))
            med = [sorted(r[i] for r in runs)[len(runs) // 2] for i in range(4)]
            rows.append({"U": U, "strips_of_128": (U + 128) // 128, "lattice_us": round(med[2], 1),
                         "forward_call_us": round(sum(med), 1),
                         "lattice_ns_per_diagonal": round(med[2] * 1e3 / (Tl + U), 1)})
            del xl, yl, cl, stl
        result["long_labels"] = {"N": 4, "T": 1250, "V": 4, "mode": "log-prob", "cases": rows}

    if args.with_pack:
        Tm, Up = int(cfg["lx"].max()), int(cfg["ly"].max()) + 1
        x4 = torch.zeros((N, Tm, Up, V), dtype=tdt, device=dev)
        packed = pkg.pack_padded(x4, lx, ly, total_rows=R)
        lib = pkg._lib.load()
        row_off, _st = pkg.loss._offsets(lx, ly, R)
        g4 = torch.empty_like(x4)
        dt = pkg.loss._DTYPES[tdt]
        stream = torch.cuda.current_stream().cuda_stream
        pack_ms = timed(lambda: lib.cwr_pack(x4.data_ptr(), dt, N, Tm, Up, V, lx.data_ptr(), ly.data_ptr(),
                                             row_off.data_ptr(), R, packed.data_ptr(), None, stream))
        unpack_ms = timed(lambda: lib.cwr_unpack(packed.data_ptr(), dt, N, Tm, Up, V, lx.data_ptr(), ly.data_ptr(),
                                                 row_off.data_ptr(), R, g4.data_ptr(), stream))
        padded_bytes = x4.numel() * esize
        result["pack_op"] = {
            "padded_shape": [N, Tm, Up, V], "pack_ms": round(pack_ms, 4), "unpack_ms": round(unpack_ms, 4),
            # pack: read + write the R valid rows; unpack: read them, write every padded row
            "pack_GBs": round(2 * R * V * esize / (pack_ms * 1e-3) / 1e9, 1),
            "unpack_GBs": round((R * V * esize + padded_bytes) / (unpack_ms * 1e-3) / 1e9, 1)}
        del x4, g4, packed

    if args.with_joiner:
        H = 512
        lib = pkg._lib.load()
        Tm, Up = int(cfg["lx"].max()), int(cfg["ly"].max()) + 1
        f = torch.randn((N, Tm, H), device=dev).to(tdt)
        g = torch.randn((N, Up, H), device=dev).to(tdt)
        row_off, _st = pkg.loss._offsets(lx, ly, R)
        h = torch.empty((R, H), dtype=tdt, device=dev)
        dh = torch.randn((R, H), device=dev).to(tdt)
        df, dg = torch.empty_like(f), torch.empty_like(g)
        dt = pkg.loss._DTYPES[tdt]
        stream = torch.cuda.current_stream().cuda_stream
        ops = {}
        for name, act in (("sum", 0), ("tanh", 1)):
            fw = timed(lambda: lib.cwr_join(f.data_ptr(), g.data_ptr(), dt, act, N, Tm, Up, H, lx.data_ptr(),
                                            ly.data_ptr(), row_off.data_ptr(), R, h.data_ptr(), None, stream))
            bw = timed(lambda: lib.cwr_join_backward(dh.data_ptr(), h.data_ptr(), dt, act, N, Tm, Up, H,
                                                     lx.data_ptr(), ly.data_ptr(), row_off.data_ptr(), R,
                                                     df.data_ptr(), dg.data_ptr(), stream))
            rb = R * H * esize
            # forward: the (R,H) rows stored; backward: dh (and h with an activation) read once per sum
            ops[name] = {"forward_ms": round(fw, 4), "backward_ms": round(bw, 4),
                         "forward_GBs": round(rb / (fw * 1e-3) / 1e9, 1),
                         "backward_GBs": round((2 if act == 0 else 4) * rb / (bw * 1e-3) / 1e9, 1)}
        result["joiner_op"] = {"H": H, "rows": R, **ops}
        del f, g, h, dh, df, dg

    if args.with_fused_joiner:
        # The output layer fused into the loss (cwr_joint_forward / cwr_joint_backward) on this config's
        # lengths: bf16 (R,H) x (H,V) on the matrix cores.  Algorithmic flops: 2 R H V forward, 6 R H V
        # forward + backward (logits, dh, dW); the logits formed a second time in the backward pass
        # are not counted.  Beside it the route through stored logits: library GEMM, then the fused
        # loss over the (R,V) bf16 logits (three passes over them).
        H = args.joint_dim
        jd = torch.bfloat16
        hj = torch.randn((R, H), device=dev).to(jd)
        Wj = (torch.randn((V, H), device=dev) / H ** 0.5).to(jd)
        bj = torch.randn(V, device=dev).to(jd)
        lib = pkg._lib.load()
        stream = torch.cuda.current_stream().cuda_stream
        flops = 2.0 * R * H * V
        fwd_call = timed(lambda: pkg.joint_forward(hj, Wj, bj, lx, y, ly, 0, max_u=y.size(1)))
        _c, jst = pkg.joint_forward(hj, Wj, bj, lx, y, ly, 0, max_u=y.size(1))
        b32 = bj.float()
        dzb = torch.empty((R, V), dtype=jd, device=dev)
        dz_ms = timed(lambda: lib.cwr_joint_backward(
            hj.data_ptr(), Wj.data_ptr(), b32.data_ptr(), pkg.loss._DTYPES[jd], R, H, V, N, 0, jst.rowinfo.data_ptr(),
            jst.grads.data_ptr(), jst.lse.data_ptr(), go.data_ptr(), 1, 1.0, dzb.data_ptr(), stream))
        del dzb, jst
        hp, Wp, bp = (t.clone().requires_grad_(True) for t in (hj, Wj, bj))

        def fused_step():
            hp.grad = Wp.grad = bp.grad = None
            pkg.fused_joint_loss(hp, Wp, bp, lx, y, ly, 0, "mean", max_u=y.size(1)).backward()

        def stored_step():
            hp.grad = Wp.grad = bp.grad = None
            z = torch.nn.functional.linear(hp, Wp, bp)
            pkg.transducer_loss(z, lx, y, ly, 0, "mean", fused_log_softmax=True, max_u=y.size(1)).backward()

        def stored_fwd():
            with torch.no_grad():
                z = torch.nn.functional.linear(hj, Wj, bj)
            pkg.rnnt_forward(z, lx, y, ly, 0, True, max_u=y.size(1))

        joiner_chain = None  # the one-kernel form exists for the joint sizes whose rows stay in registers
        if H in pkg.loss.RESIDENT_JOINT_SIZES:
            # The joiner's whole chain (broadcast sum + tanh + output layer + loss) as one kernel against
            # its two-kernel form (cwr_join, then cwr_joint_forward on the stored rows), same lengths.
            Tm, Up = int(cfg["lx"].max()), int(cfg["ly"].max()) + 1
            fj = torch.randn((N, Tm, H), device=dev).to(jd)
            gj = torch.randn((N, Up, H), device=dev).to(jd)
            chain_fwd = timed(lambda: pkg.loss.joint_forward_fg(fj, gj, 1, Wj, bj, lx, y, ly, 0, R, max_u=y.size(1)))
            chain_fwd_keep = timed(lambda: pkg.loss.joint_forward_fg(fj, gj, 1, Wj, bj, lx, y, ly, 0, R, max_u=y.size(1),
                                                                     keep_rows=True))

            def two_kernel_fwd():
                hh = pkg.compact_join(fj, gj, lx, ly, "tanh", total_rows=R)
                pkg.joint_forward(hh, Wj, bj, lx, y, ly, 0, max_u=y.size(1))

            two_fwd = timed(two_kernel_fwd)
            fp, gp = fj.clone().requires_grad_(True), gj.clone().requires_grad_(True)

            def chain_step():
                fp.grad = gp.grad = Wp.grad = bp.grad = None
                pkg.fused_joiner_loss(fp, gp, Wp, bp, lx, y, ly, 0, "mean", "tanh", total_rows=R, max_u=y.size(1),
                                      one_kernel=True).backward()

            def two_kernel_step():
                fp.grad = gp.grad = Wp.grad = bp.grad = None
                hh = pkg.compact_join(fp, gp, lx, ly, "tanh", total_rows=R)
                pkg.fused_joint_loss(hh, Wp, bp, lx, y, ly, 0, "mean", max_u=y.size(1)).backward()

            chain_ms = timed(chain_step)
            two_ms = timed(two_kernel_step)
            joiner_chain = {"what": "act(f[n,t] + g[n,u]) @ W^T + bias -> loss, tanh, f (N,T,H), g (N,U+1,H)",
                            "forward_one_kernel_ms": round(chain_fwd, 4),
                            "forward_one_kernel_keeping_rows_ms": round(chain_fwd_keep, 4),
                            "forward_join_then_joint_ms": round(two_fwd, 4),
                            "fwd_bwd_one_kernel_forward_ms": round(chain_ms, 4),
                            "fwd_bwd_join_then_joint_ms": round(two_ms, 4)}
            del fj, gj, fp, gp

        torch.cuda.reset_peak_memory_stats()
        base_mem = torch.cuda.memory_allocated()
        fused_ms = timed(fused_step)
        fused_mem = torch.cuda.max_memory_allocated() - base_mem
        torch.cuda.reset_peak_memory_stats()
        stored_ms = timed(stored_step)
        stored_mem = torch.cuda.max_memory_allocated() - base_mem
        stored_fwd_ms = timed(stored_fwd)
        result["fused_joiner"] = {
            "H": H, "rows": R, "V": V, "dtype": "bf16", "peak_TFLOPs": MFMA_BF16_PEAK_TFLOPS,
            "forward_call_ms": round(fwd_call, 4),
            "forward_TFLOPs": round(flops / (fwd_call * 1e-3) / 1e12, 1),
            "dlogits_kernel_ms": round(dz_ms, 4),
            "dlogits_TFLOPs": round(flops / (dz_ms * 1e-3) / 1e12, 1),
            # the one matrix-core kernel launched alone here: logits formed on MFMA (2 R H V flops per
            # launch), turned into their gradient in registers and stored
            "roofline": {"bound": "mfma", "kernel": "k_joint_dz (cwr_joint_backward)",
                         "achieved": round(flops / (dz_ms * 1e-3) / 1e12, 1), "peak": MFMA_BF16_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(flops / (dz_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)},
            "fwd_bwd_ms": round(fused_ms, 4),
            "fwd_bwd_TFLOPs": round(3 * flops / (fused_ms * 1e-3) / 1e12, 1),
            "fwd_bwd_frac_of_peak": round(3 * flops / (fused_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
            "fwd_bwd_peak_extra_MiB": round(fused_mem / 2 ** 20, 1),
            "joiner_chain": joiner_chain,
            "stored_logits_route": {"what": "torch linear (library GEMM) + transducer_loss(fused_log_softmax=True)",
                                    "forward_ms": round(stored_fwd_ms, 4), "fwd_bwd_ms": round(stored_ms, 4),
                                    "fwd_bwd_peak_extra_MiB": round(stored_mem / 2 ** 20, 1)}}
        del hj, Wj, bj, hp, Wp, bp

    if not args.no_cpu:
        g_all = pkg.rnnt_backward(xd, lx, y, ly, 0, st, go, out=out)
        torch.cuda.synchronize()
        dev_out = {"costs": costs.double().cpu().numpy(),
                   "grad": lambda a, b: g_all[a:b].double().cpu().numpy()}
        base, parity = cpu_baseline(cfg, x_cpu, args.cpu_budget, dev_out)
        base["value"] = round(base["value"], 4)
        result["cpu_baseline"] = base
        result["parity"] = parity
        try:
            import torchaudio  # noqa: F401
            result["cpu_baseline"]["torchaudio"] = "installed but not used by this leg"
        except Exception:
            result["cpu_baseline"]["torchaudio"] = "n/a (not installed)"
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
