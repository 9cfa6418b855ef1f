#!/usr/bin/env python3
"""Per-kernel roofline measurements through the C ABI (no model around the kernels).

    python -m cavs_amd.kernel_bench [--set copies|gemm|gates|rounds|tails|all] [--iters 50]

For each case: launches the entry point `iters` times back to back on one stream between two
HIP events (launches shorter than 12 us: timed one at a time by the events their own kernels
stamp) and reports the average duration per launch, the algorithmic bytes / flops
per launch and the fraction of the MI355X roofline (HBM 8 TB/s, FP32 MFMA 157.3 TFLOP/s).
Shapes are the ones the benchmark configurations produce (C3: H=512, C5: H=1024).
One JSON object per line.
"""
import argparse
import ctypes as C
import json

import torch

from . import hip

HBM_GBS = 8000.0
MFMA_TF = 157.3


_last_timing = "back to back"


def _time(fn, iters, stream):
    global _last_timing
    _last_timing = "back to back"
    e0, e1 = C.c_void_p(), C.c_void_p()
    hip.call("cavs_event_create", C.byref(e0))
    hip.call("cavs_event_create", C.byref(e1))
    for _ in range(3):
        fn()
    hip.call("cavs_stream_sync", stream)
    hip.call("cavs_event_record", e0, stream)
    for _ in range(iters):
        fn()
    hip.call("cavs_event_record", e1, stream)
    ms = C.c_float()
    hip.call("cavs_event_elapsed_ms", C.byref(ms), e0, e1)
    us = ms.value * 1e3 / iters  # us per launch
    if us < 12.0:
        # A call from Python costs about 6 us, so a loop of short launches times the host.  Such a
        # launch is timed by the events its own kernels stamp (first kernel's start to last kernel's
        # end, the interval a kernel trace reports), behind three launches that keep the queue busy.
        total, launched = 0.0, C.c_int()
        for _ in range(iters):
            for _ in range(3):
                fn()
            hip.call("cavs_profile_arm", e0, e1)
            fn()
            hip.call("cavs_profile_disarm", C.byref(launched))
            hip.call("cavs_event_elapsed_ms", C.byref(ms), e0, e1)
            total += ms.value
        us = total * 1e3 / iters
        _last_timing = "kernel-stamped"
    hip.call("cavs_event_destroy", e0)
    hip.call("cavs_event_destroy", e1)
    return us


def _emit(kernel, shape, us, nbytes=None, flops=None):
    rec = dict(kernel=kernel, shape=shape, us_per_launch=round(us, 3), timing=_last_timing)
    if nbytes is not None:
        gbs = nbytes / us / 1e3
        rec.update(bound="hbm", bytes_per_launch=int(nbytes), achieved_GBs=round(gbs, 1),
                   frac=round(gbs / HBM_GBS, 4))
    if flops is not None:
        tf = flops / us / 1e6
        rec.update(bound="mfma", flops_per_launch=int(flops), achieved_TFLOPs=round(tf, 2),
                   frac=round(tf / MFMA_TF, 4))
    print(json.dumps(rec), flush=True)


def copies(iters, st):
    f32 = dict(dtype=torch.float32, device="cuda")
    for n, w, tag in [(600, 1024, "C3 round"), (2482, 1024, "C3 all rows"), (16384, 2048, "C5 round"),
                      (65536, 2048, "C5 leaf round"), (131072, 1024, "wide batch")]:
        rows = 2 * n
        src = torch.randn(rows, w, **f32)
        out = torch.empty(n, w, **f32)
        g = torch.Generator(device="cpu").manual_seed(n)
        ids = torch.randperm(rows, generator=g)[:n].to(torch.int32).cuda()
        nbytes = n * (8 * w + 4)
        us = _time(lambda: hip.call("cavs_gather_rows", out.data_ptr(), w, src.data_ptr(), w, ids.data_ptr(),
                                    n, w, st), iters, st)
        _emit("gather_rows", f"{tag}: n={n} w={w}", us, nbytes=nbytes)
        dst = torch.empty(rows, w, **f32)
        us = _time(lambda: hip.call("cavs_scatter_rows", dst.data_ptr(), w, ids.data_ptr(), out.data_ptr(), w,
                                    n, w, st), iters, st)
        _emit("scatter_rows", f"{tag}: n={n} w={w}", us, nbytes=nbytes)
        us = _time(lambda: hip.call("cavs_copy_rows", out.data_ptr(), w, src.data_ptr(), w, n, w, st), iters, st)
        _emit("copy_rows", f"{tag}: n={n} w={w}", us, nbytes=n * 8 * w)
        if n % 2 == 0:
            m = n // 2
            G = torch.empty(2 * m, w, **f32)
            hs = torch.empty(m, w // 2, **f32)
            us = _time(lambda: hip.call("cavs_gather_children", G.data_ptr(), hs.data_ptr(), src.data_ptr(),
                                        ids.data_ptr(), m, w, w // 2, st), iters, st)
            _emit("gather_children", f"{tag}: vertices={m} w={w}", us, nbytes=2 * m * (8 * w + 4) + 4 * m * (w // 2))


def gemm(iters, st):
    f32 = dict(dtype=torch.float32, device="cuda")
    cases = []
    for H, E, N, tag in [(512, 300, 2482, "C3"), (1024, 1024, 73000, "C5")]:
        n = 600 if H == 512 else 16384
        cases += [
            (0, 0, N, 4 * H, E, f"{tag} x*W all rows"),
            (0, 0, n, 3 * H, H, f"{tag} round h_lr*U_iou"),
            (0, 0, 2 * n, H, H, f"{tag} round [h_l;h_r]*U_f"),
            (0, 1, n, H, 3 * H, f"{tag} round d(hU)*U_iou^T"),
            (0, 1, 2 * n, H, H, f"{tag} round dF*U_f^T"),
            (0, 1, N, E, 4 * H, f"{tag} de = dxW*W^T"),
            (1, 0, E, 4 * H, N, f"{tag} dW = e^T*dxW"),
            (1, 0, H, 3 * H, N // 2, f"{tag} dU_iou = h_lr^T*d(hU)"),
        ]
    cases += [(0, 0, 32, 1536, 512, "C3 tail round (32 rows)"), (0, 0, 8192, 8192, 8192, "square 8192")]
    # the 10000-way head of the variable-length LSTM configuration (7331 tokens per batch) in the forms the
    # engine runs: the weights Wc [C, H] are read through their [H, C] copy
    cases += [(0, 0, 7331, 10000, 512, "C4 head logits = h*WcT"), (1, 0, 10000, 512, 7331, "C4 head dWc = dlogits^T*h"),
              (0, 1, 7331, 512, 10000, "C4 head dh = dlogits*WcT^T"), (0, 0, 7331, 2048, 512, "C4 x*W all rows"),
              # (the same two products on Wc itself, as they ran before the copy)
              (0, 1, 7331, 10000, 512, "C4 head logits = h*Wc^T, on Wc"), (0, 0, 7331, 512, 10000, "C4 head dh = dlogits*Wc, on Wc")]
    # what the matrix pipes sustain with register operands only, in launches of ~1 ms and ~10 ms
    buf = torch.empty(1 << 20, **f32)
    for mf_iters in (4000, 40000):
        fl = C.c_double()
        us = _time(lambda: hip.call("cavs_mfma_probe", buf.data_ptr(), buf.numel(), mf_iters, C.byref(fl), st), max(iters // 10, 3), st)
        _emit("mfma_probe", f"register operands only, {mf_iters} x 8 MFMA 32x32x2 per wavefront, 4 workgroups per CU", us, flops=fl.value)
    for tA, tB, M, Nn, K, tag in cases:
        A = torch.randn((K, M) if tA else (M, K), **f32)
        B = torch.randn((Nn, K) if tB else (K, Nn), **f32)
        Cm = torch.empty(M, Nn, **f32)
        nb = hip.lib().cavs_sgemm_splitk_workspace(M, Nn, K)
        ws = torch.empty(max(nb // 4, 4), **f32)
        us = _time(lambda: hip.call("cavs_sgemm_splitk", tA, tB, M, Nn, K, 1.0, A.data_ptr(), A.shape[1],
                                    B.data_ptr(), B.shape[1], 0.0, Cm.data_ptr(), Nn, ws.data_ptr(), nb, st),
                   max(5, iters // 5) if M * Nn * K > 1e11 else iters, st)
        _emit("sgemm", f"{tag}: {'T' if tA else 'N'}{'T' if tB else 'N'} M={M} N={Nn} K={K}", us,
              flops=2.0 * M * Nn * K)
        del A, B, Cm, ws
    # the once-per-step products of a C3 batch as one grouped launch
    H, E, N = 512, 300, 2482
    shapes = [(0, 1, N, E, 4 * H), (1, 0, E, 4 * H, N), (1, 0, H, 3 * H, N // 2), (1, 0, H, H, N)]
    descs = (hip.GemmDesc * len(shapes))()
    keep = []
    for p, (tA, tB, M, Nn, K) in enumerate(shapes):
        A = torch.randn((K, M) if tA else (M, K), **f32)
        B = torch.randn((Nn, K) if tB else (K, Nn), **f32)
        Cm = torch.empty(M, Nn, **f32)
        keep += [A, B, Cm]
        descs[p] = hip.GemmDesc(tA, tB, M, Nn, K, 1.0, 0.0, A.data_ptr(), A.shape[1], B.data_ptr(), B.shape[1],
                                Cm.data_ptr(), Nn)
    nb = hip.lib().cavs_sgemm_group_workspace(len(shapes), descs)
    ws = torch.empty(max(nb // 4, 4), **f32)
    us = _time(lambda: hip.call("cavs_sgemm_group", len(shapes), descs, ws.data_ptr(), nb, st), iters, st)
    _emit("sgemm_group", "C3 step: de + dW + dU_iou + dU_f in one launch (+ one reduce)", us,
          flops=sum(2.0 * M * Nn * K for _, _, M, Nn, K in shapes))
    del keep, ws
    # C5's de with the block hint of a step: the first half of the slab rows are leaves, whose forget-gate
    # columns of dxW are zero; the flops are those left to do
    H, E, N = 1024, 1024, 73000
    A, B, Cm = torch.randn(N, 4 * H, **f32), torch.randn(E, 4 * H, **f32), torch.empty(N, E, **f32)
    A[:N // 2, 3 * H:] = 0
    one = (hip.GemmDesc * 1)()
    one[0] = hip.GemmDesc(0, 1, N, E, 4 * H, 1.0, 0.0, A.data_ptr(), 4 * H, B.data_ptr(), 4 * H, Cm.data_ptr(), E, hip.GEMM_A_ZERO, N // 2, 3 * H)
    us = _time(lambda: hip.call("cavs_sgemm_group", 1, one, None, 0, st), max(5, iters // 5), st)
    _emit("sgemm_group", f"C5 de = dxW*W^T, f columns of {N // 2} leaf rows known zero: NT M={N} N={E} K={4 * H}", us,
          flops=2.0 * N * E * 4 * H - 2.0 * (N // 2) * E * H)


def gates(iters, st):
    f32 = dict(dtype=torch.float32, device="cuda")
    for n, H, tag in [(600, 512, "C3 round"), (16384, 1024, "C5 round")]:
        xW, hU, hUf = torch.randn(n, 4 * H, **f32), torch.randn(n, 3 * H, **f32), torch.randn(2 * n, H, **f32)
        G, bias = torch.randn(2 * n, 2 * H, **f32), torch.randn(4 * H, **f32)
        gt, msg = torch.empty(n, 6 * H, **f32), torch.empty(n, 2 * H, **f32)
        us = _time(lambda: hip.call("cavs_treelstm_gates_fwd", xW.data_ptr(), 4 * H, hU.data_ptr(), hUf.data_ptr(),
                                    G.data_ptr(), bias.data_ptr(), gt.data_ptr(), msg.data_ptr(), n, H, st), iters, st)
        _emit("treelstm_gates_fwd", f"{tag}: n={n} H={H}", us, nbytes=4 * n * H * 21 + 16 * H)
        dmsg, dret = torch.randn(n, 2 * H, **f32), torch.randn(n, H, **f32)
        dxW, dF, dG = torch.empty(n, 4 * H, **f32), torch.empty(2 * n, H, **f32), torch.empty(2 * n, 2 * H, **f32)
        us = _time(lambda: hip.call("cavs_treelstm_gates_bwd", dmsg.data_ptr(), dret.data_ptr(), gt.data_ptr(),
                                    G.data_ptr(), dxW.data_ptr(), 4 * H, dF.data_ptr(), dG.data_ptr(), n, H, st),
                   iters, st)
        # reads dmsg 2H, dret H, gates 6H, c_l c_r 2H; writes dxW 4H, dF 2H, dc_l dc_r 2H
        _emit("treelstm_gates_bwd", f"{tag}: n={n} H={H}", us, nbytes=4 * n * H * 19)


def rounds(iters, st):
    """One Tree-LSTM round as fused launches, beside the same round as separate launches."""
    f32 = dict(dtype=torch.float32, device="cuda")
    for n, H, tag in [(4, 512, "C3 tail"), (16, 512, "C3 tail"), (32, 512, "C3 tail"), (64, 512, "C3 tail"),
                      (150, 512, "C3 mid"), (300, 512, "C3 mid"), (600, 512, "C3 mid"), (1200, 512, "2x C3"),
                      (2400, 512, "4x C3"), (2048, 1024, "C5 small round")]:
        rows = 3 * n
        pool = torch.randn(rows, 2 * H, **f32) * 0.5
        g = torch.Generator(device="cpu").manual_seed(n)
        child = torch.randperm(2 * n, generator=g).to(torch.int32).cuda()
        pair = (2 * n + torch.arange(n)).to(torch.int32).cuda()
        xW, bias = torch.randn(n, 4 * H, **f32), torch.randn(4 * H, **f32)
        U = torch.randn(4 * H * H, **f32) / H ** 0.5
        G, hlr = torch.empty(2 * n, 2 * H, **f32), torch.empty(n, H, **f32)
        gt, msg = torch.empty(n, 6 * H, **f32), torch.empty(n, 2 * H, **f32)
        flops = 2.0 * n * H * 5 * H
        us = _time(lambda: hip.call("cavs_treelstm_round_fwd", pool.data_ptr(), child.data_ptr(), pair.data_ptr(),
                                    xW.data_ptr(), 4 * H, U.data_ptr(), bias.data_ptr(), G.data_ptr(), hlr.data_ptr(),
                                    gt.data_ptr(), msg.data_ptr(), None, None, n, H, st), iters, st)
        _emit("treelstm_round_fwd", f"{tag}: n={n} H={H}", us, flops=flops)
        if hip.lib().cavs_round_packed_ok(n, H):  # the same launch reading U from its tile-major copy
            Upk = torch.empty(4 * H * H, **f32)
            T = hip.Task
            jobs = [T(hip.TASK_SGD_PACK, 0.0, H, 3 * H, 0, Upk.data_ptr(), U.data_ptr(), None, None),
                    T(hip.TASK_SGD_PACK, 0.0, H, H, 0, Upk.data_ptr() + 4 * 3 * H * H, U.data_ptr() + 4 * 3 * H * H, None, None)]
            hip.call("cavs_run_tasks", len(jobs), (T * len(jobs))(*jobs), st)
            us = _time(lambda: hip.call("cavs_treelstm_round_fwd_packed", pool.data_ptr(), child.data_ptr(), pair.data_ptr(),
                                        xW.data_ptr(), 4 * H, U.data_ptr(), Upk.data_ptr(), bias.data_ptr(), G.data_ptr(),
                                        hlr.data_ptr(), gt.data_ptr(), msg.data_ptr(), None, None, n, H, st), iters, st)
            _emit("treelstm_round_fwd_packed", f"{tag}: n={n} H={H}", us, flops=flops)
            del Upk
        hU, hUf = torch.empty(n, 3 * H, **f32), torch.empty(2 * n, H, **f32)

        def separate_fwd():
            hip.call("cavs_gather_children", G.data_ptr(), hlr.data_ptr(), pool.data_ptr(), child.data_ptr(), n, 2 * H, H, st)
            hip.call("cavs_sgemm", 0, 0, n, 3 * H, H, 1.0, hlr.data_ptr(), H, U.data_ptr(), 3 * H, 0.0, hU.data_ptr(), 3 * H, st)
            hip.call("cavs_sgemm", 0, 0, 2 * n, H, H, 1.0, G.data_ptr(), 2 * H, U.data_ptr() + 4 * 3 * H * H, H, 0.0,
                     hUf.data_ptr(), H, st)
            hip.call("cavs_treelstm_gates_fwd", xW.data_ptr(), 4 * H, hU.data_ptr(), hUf.data_ptr(), G.data_ptr(),
                     bias.data_ptr(), gt.data_ptr(), msg.data_ptr(), n, H, st)
            hip.call("cavs_scatter_rows", pool.data_ptr(), 2 * H, pair.data_ptr(), msg.data_ptr(), 2 * H, n, 2 * H, st)

        us = _time(separate_fwd, iters, st)
        _emit("round fwd as 5 launches", f"{tag}: n={n} H={H}", us, flops=flops)
        UT = torch.empty(4 * H * H, **f32)
        hip.call("cavs_transpose", UT.data_ptr(), U.data_ptr(), H, 3 * H, st)
        hip.call("cavs_transpose", UT.data_ptr() + 4 * 3 * H * H, U.data_ptr() + 4 * 3 * H * H, H, H, st)
        dpool, dret = torch.randn(rows, 2 * H, **f32), torch.randn(n, H, **f32)
        dxW, dF = torch.empty(n, 4 * H, **f32), torch.empty(2 * n, H, **f32)
        us = _time(lambda: hip.call("cavs_treelstm_round_bwd_gates", dpool.data_ptr(), pair.data_ptr(), child.data_ptr(),
                                    dret.data_ptr(), None, gt.data_ptr(), G.data_ptr(), dxW.data_ptr(), 4 * H, dF.data_ptr(),
                                    n, H, st), iters, st)
        # reads dmsg 2H, dret H, gates 6H, c_l c_r 2H; writes dxW 4H, dF 2H, dc_l dc_r 2H
        _emit("treelstm_round_bwd_gates", f"{tag}: n={n} H={H}", us, nbytes=4 * n * H * 19)
        us = _time(lambda: hip.call("cavs_treelstm_round_bwd_children", dxW.data_ptr(), 4 * H, dF.data_ptr(), UT.data_ptr(),
                                    child.data_ptr(), dpool.data_ptr(), n, H, st), iters, st)
        _emit("treelstm_round_bwd_children", f"{tag}: n={n} H={H}", us, flops=flops)
        # the backward round as the engine launches it when the batch's message flow is a forest: the
        # children's d h and their gate gradients in one launch, transposed weights tile-major.
        # Whole-batch slabs of 3n rows: the round is rows [2n, 3n), its children rows [0, 2n)
        if hip.lib().cavs_round_packed_ok(n, H):
            R3 = 3 * n
            UTp = torch.empty(4 * H * H, **f32)
            tasks = (hip.Task * 2)(hip.Task(hip.TASK_PACK_T, 0.0, H, 3 * H, 0, UTp.data_ptr(), U.data_ptr(), None, None),
                                   hip.Task(hip.TASK_PACK_T, 0.0, H, H, 0, UTp.data_ptr() + 4 * 3 * H * H,
                                            U.data_ptr() + 4 * 3 * H * H, None, None))
            hip.call("cavs_run_tasks", 2, tasks, st)
            dxW_all, dF_all, dc_all = torch.randn(R3, 4 * H, **f32), torch.randn(2 * R3, H, **f32), torch.randn(R3, H, **f32)
            gates_all, G_all = torch.rand(R3, 6 * H, **f32), torch.randn(2 * R3, 2 * H, **f32)
            dgo = torch.randn(R3, H, **f32)
            rows_all = torch.arange(R3, dtype=torch.int32, device="cuda")
            kids = torch.randperm(2 * n, generator=torch.Generator(device="cpu").manual_seed(n)).to(torch.int32).cuda()
            us = _time(lambda: hip.call("cavs_treelstm_round_bwd_children_gates_packed", dxW_all.data_ptr(), 4 * H, dF_all.data_ptr(),
                                        dc_all.data_ptr(), UTp.data_ptr(), kids.data_ptr(), gates_all.data_ptr(), G_all.data_ptr(),
                                        dgo.data_ptr(), rows_all.data_ptr(), 2 * n, n, n, H, st), iters, st)
            _emit("treelstm_round_bwd_children_gates_packed", f"{tag}: n={n} H={H}", us, flops=flops)
            del UTp, dxW_all, dF_all, dc_all, gates_all, G_all, dgo
        del pool, xW, U, G, hlr, gt, msg, hU, hUf, UT, dpool, dret, dxW, dF


def tails(iters, st):
    """The rounds near the roots of a Tree-LSTM batch (H = 512) as one launch per direction, beside the
    same rounds as one packed launch each.  The batch: 8 x `width` complete binary trees side by
    side, rounds of 8 * width, 4 * width ... 8 rows above 16 * width leaf rows; a group runs `width` trees."""
    import numpy as np
    f32 = dict(dtype=torch.float32, device="cuda")
    H = 512
    for width in (8, 32):
        sizes = []
        n = 8 * width
        while n >= 8:
            sizes.append(n)
            n //= 2
        leaves = 2 * sizes[0]
        offs = np.concatenate([[leaves], leaves + np.cumsum(sizes)[:-1]]).astype(np.int64)
        N = int(leaves + sum(sizes))
        child = np.full(2 * N, -1, np.int32)
        for r, (off, nr) in enumerate(zip(offs, sizes)):
            below = 0 if r == 0 else offs[r - 1]
            i = np.arange(nr)
            child[2 * (off + i)] = below + 2 * i
            child[2 * (off + i) + 1] = below + 2 * i + 1
        # group g: the rows i with i * 8 // nr == g of every round, round by round
        rows, start, count = [], np.zeros((8, len(sizes)), np.int32), np.zeros((8, len(sizes)), np.int32)
        for g in range(8):
            for r, (off, nr) in enumerate(zip(offs, sizes)):
                mine = off + np.arange(g * nr // 8, (g + 1) * nr // 8)
                start[g, r], count[g, r] = len(rows), len(mine)
                rows.extend(mine.tolist())
        nrounds = np.full(8, len(sizes), np.int32)
        flags = np.tile(np.arange(len(sizes), dtype=np.int32) * 2 + 1, (8, 1)).astype(np.int32)  # wait for the lists before, arrive
        bstart, bcount = np.ascontiguousarray(start[:, ::-1]), np.ascontiguousarray(count[:, ::-1])
        d_rows = torch.tensor(rows, dtype=torch.int32, device="cuda")
        d_child = torch.from_numpy(child).cuda()
        d_pair = torch.arange(N, dtype=torch.int32, device="cuda")
        pool = torch.randn(N, 2 * H, **f32) * 0.5
        xW, bias = torch.randn(N, 4 * H, **f32), torch.zeros(4 * H, **f32)
        U = torch.randn(4 * H * H, **f32) / H ** 0.5
        Upk, UTp = torch.empty(4 * H * H, **f32), torch.empty(4 * H * H, **f32)
        T = hip.Task
        jobs = [T(hip.TASK_SGD_PACK, 0.0, H, 3 * H, 0, Upk.data_ptr(), U.data_ptr(), None, None),
                T(hip.TASK_SGD_PACK, 0.0, H, H, 0, Upk.data_ptr() + 4 * 3 * H * H, U.data_ptr() + 4 * 3 * H * H, None, None),
                T(hip.TASK_PACK_T, 0.0, H, 3 * H, 0, UTp.data_ptr(), U.data_ptr(), None, None),
                T(hip.TASK_PACK_T, 0.0, H, H, 0, UTp.data_ptr() + 4 * 3 * H * H, U.data_ptr() + 4 * 3 * H * H, None, None)]
        hip.call("cavs_run_tasks", len(jobs), (T * len(jobs))(*jobs), st)
        G, hlr = torch.zeros(2 * N, 2 * H, **f32), torch.zeros(N, H, **f32)
        gt, go = torch.rand(N, 6 * H, **f32), torch.zeros(N, H, **f32)
        d_out = torch.arange(N, dtype=torch.int32, device="cuda")
        sync = torch.zeros(hip.lib().cavs_tail_sync_bytes() // 4, dtype=torch.int32, device="cuda")
        M = len(sizes)
        flops = 2.0 * sum(sizes) * H * 5 * H
        tag = f"rounds of {sizes[0]} .. {sizes[-1]} rows ({sum(sizes)} vertices), 8 groups, H={H}"

        def fwd_tail():
            hip.call("cavs_treelstm_tail_fwd", pool.data_ptr(), d_child.data_ptr(), d_pair.data_ptr(), xW.data_ptr(), 4 * H, Upk.data_ptr(),
                     bias.data_ptr(), G.data_ptr(), hlr.data_ptr(), gt.data_ptr(), None, go.data_ptr(), d_out.data_ptr(), d_rows.data_ptr(),
                     8, nrounds.ctypes.data, start.ctypes.data, count.ctypes.data, flags.ctypes.data, M, H, sync.data_ptr(), 1 << 20, 0, st)

        def fwd_rounds():
            for off, nr in zip(offs.tolist(), sizes):
                hip.call("cavs_treelstm_round_fwd_packed", pool.data_ptr(), d_child.data_ptr() + 8 * off, d_pair.data_ptr() + 4 * off,
                         xW.data_ptr() + 16 * off * H, 4 * H, U.data_ptr(), Upk.data_ptr(), bias.data_ptr(), G.data_ptr() + 16 * off * H,
                         hlr.data_ptr() + 4 * off * H, gt.data_ptr() + 24 * off * H, None, go.data_ptr(), d_out.data_ptr() + 4 * off, nr, H, st)

        us = _time(fwd_tail, iters, st)
        _emit("treelstm_tail_fwd", tag, us, flops=flops)
        us = _time(fwd_rounds, iters, st)
        _emit(f"the same as {M} cavs_treelstm_round_fwd_packed", tag, us, flops=flops)
        Gv = torch.randn(2 * N, 2 * H, **f32) * 0.5
        dgo = torch.randn(N, H, **f32)
        dxW, dF, dc = torch.zeros(N, 4 * H, **f32), torch.zeros(2 * N, H, **f32), torch.zeros(N, H, **f32)

        def bwd_tail():
            hip.call("cavs_treelstm_tail_bwd", dxW.data_ptr(), 4 * H, dF.data_ptr(), dc.data_ptr(), UTp.data_ptr(), d_child.data_ptr(),
                     gt.data_ptr(), Gv.data_ptr(), dgo.data_ptr(), d_out.data_ptr(), leaves, d_rows.data_ptr(), 8, nrounds.ctypes.data,
                     bstart.ctypes.data, bcount.ctypes.data, flags.ctypes.data, M, H, sync.data_ptr(), 1 << 20, 0, st)

        def bwd_rounds():
            for off, nr in zip(offs.tolist()[::-1], sizes[::-1]):
                hip.call("cavs_treelstm_round_bwd_children_gates_packed", dxW.data_ptr(), 4 * H, dF.data_ptr(), dc.data_ptr(), UTp.data_ptr(),
                         d_child.data_ptr() + 8 * off, gt.data_ptr(), Gv.data_ptr(), dgo.data_ptr(), d_out.data_ptr(), off, nr, leaves, H, st)

        us = _time(bwd_tail, iters, st)
        _emit("treelstm_tail_bwd", tag, us, flops=flops)
        us = _time(bwd_rounds, iters, st)
        _emit(f"the same as {M} cavs_treelstm_round_bwd_children_gates_packed", tag, us, flops=flops)
        assert int(sync[1].item()) == 0, "a tail launch gave up"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--set", default="all", choices=["copies", "gemm", "gates", "rounds", "tails", "all"])
    ap.add_argument("--iters", type=int, default=50)
    a = ap.parse_args()
    assert torch.cuda.is_available(), "kernel_bench needs the MI355X"
    hip.call("cavs_init", 0)
    st = torch.cuda.current_stream().cuda_stream
    if a.set in ("copies", "all"):
        copies(a.iters, st)
    if a.set in ("gemm", "all"):
        gemm(a.iters, st)
    if a.set in ("gates", "all"):
        gates(a.iters, st)
    if a.set in ("rounds", "all"):
        rounds(a.iters, st)
    if a.set in ("tails", "all"):
        tails(a.iters, st)


if __name__ == "__main__":
    main()
