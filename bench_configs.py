#!/usr/bin/env python3
"""Per-GEMM timings of the five workload configurations on one MI355X, plus the ops around them.

`bench.py` reports the headline metric (4096^3); this companion times every GEMM shape the configurations contain
(Linear forward / dX / dW at small f32 size, broadcast-rhs f16, attention-shaped batched f16, the encoder block's
bf16 Linears, vec.mat / mat.vec), the HBM-bound ops between them (softmax, bias, reshape, layer norm, ReLU, add), one
whole encoder block with every op on the device, and a few conv2d layers.  GEMMs are timed with HIP events on the library's stream (dfdx_rocm_gemm_time), the other ops with
events around a loop of calls.  One line per case on stdout; `--json FILE` also writes them as JSON.

Synthetic inputs, resident in HBM before timing.  Nothing here touches the CPU oracle.
"""
from __future__ import annotations

import argparse
import json
import sys

ROTATE_BYTES = 320 << 20   # bytes in flight across the rotating buffer sets: more than the 256 MB last-level cache


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--json", default=None, help="also write the rows to this file")
    ap.add_argument("--iters", type=int, default=30)
    ap.add_argument("--only", default="", help="comma-separated groups: c1,c3,c4,c5,fill,gemv,glue,block,conv (on request only: torch = vendor-library cross-check, edge = operands off the 16-byte grid, with the scalar kernel forced beside them, shapes = shape classes outside the configurations: few rows or columns, thin contractions, rank-1 updates, mid-size products, plancheck = the planner's pick against every forced tile variant and split count on a fixed list of shapes; exits 1 with --strict when a pick is more than --plancheck-slack off the best; fewrows = the same check on 128 products of 2 - 16 rows against matrices of 2 - 270 MB, convx = conv2d with strides, a first layer, depthwise filters, wide rows, small images in f32, 5 x 5 filters, longrows = softmax and LayerNorm on rows of 4096 - 50257 elements)")
    ap.add_argument("--strict", action="store_true", help="plancheck: exit status 1 when a pick is flagged")
    ap.add_argument("--plancheck-slack", type=float, default=0.10, help="plancheck: flag a pick that is this much slower than the best forced candidate")
    ap.add_argument("--probe", default="", choices=["", "traffic", "rows", "variants", "f32-forms", "layouts"],
                    help="counter-collection aids for rocprofv3, nothing is timed: traffic = 3 plain 256 MiB device copies (a kernel "
                         "of known size that calibrates FETCH_SIZE / WRITE_SIZE) then 5 launches of the 4096^3 f16 GEMM; rows = the same copies, then 3 launches each of "
                         "the HBM-bound rows (config 4 scores and dP, the 16384^2 f16 vec.mat and the rank-1 update that is its weight gradient, softmax forward and backward on the scores); f32-forms = 3 "
                         "launches each of the register-staged and the LDS-DMA f32 kernel (256x256 tile) on 4096^3 A.B^T and A.B; variants = 3 "
                         "launches of that GEMM with every f16 MFMA tile variant forced in turn; layouts = 5 launches each of the f16 4096^3 GEMM as "
                         "A.B^T, A.B and A^T.B, then bf16 A.B (the planner's kernel: one tile, four operand layouts)")
    ap.add_argument("--no-rotate", action="store_true", help="skip the second timing of the HBM-bound cases over rotating buffer sets")
    args = ap.parse_args()
    import torch
    from dfdx_amd import Rocm
    from dfdx_amd.rocm import GemmDesc, View

    if not torch.cuda.is_available():
        sys.exit("bench_configs.py needs a GPU")
    dev = Rocm(0)
    if args.probe:
        from dfdx_amd.rocm import KERNEL_MFMA

        n = 4096
        a = (torch.rand(n, n, device="cuda") * 2 - 1).half()
        b = (torch.rand(n, n, device="cuda") * 2 - 1).half()
        c = torch.zeros(n, n, device="cuda", dtype=torch.float16)
        if args.probe == "traffic":
            src = torch.ones(256 << 20, dtype=torch.uint8, device="cuda")
            dst = torch.empty_like(src)
            desc = dev.gemm_desc("f16", n, n, n, a.data_ptr(), (n, 1), b.data_ptr(), (n, 1), c.data_ptr(), (n, 1))
            torch.cuda.synchronize()
            for _ in range(3):
                dst.copy_(src)
            torch.cuda.synchronize()
            for _ in range(5):
                dev.gemm(desc)
            torch.cuda.synchronize()
            print(json.dumps({"probe": "3 x 256 MiB copy, 5 x " + dev.gemm_plan(desc)[2]}))
        elif args.probe == "layouts":
            names = []
            cases = [("f16", (n, 1), (1, n)), ("f16", (n, 1), (n, 1)), ("f16", (1, n), (n, 1))]
            for dt_, astr, bstr in cases:
                desc = dev.gemm_desc(dt_, n, n, n, a.data_ptr(), astr, b.data_ptr(), bstr, c.data_ptr(), (n, 1))
                names.append(dev.gemm_plan(desc)[2] + " A%s B%s" % ("" if astr[1] == 1 else "^T", "" if bstr[1] == 1 else "^T"))
                for _ in range(5):
                    dev.gemm(desc)
                torch.cuda.synchronize()
            ab, bb, cb = a.bfloat16(), b.bfloat16(), c.bfloat16()
            desc = dev.gemm_desc("bf16", n, n, n, ab.data_ptr(), (n, 1), bb.data_ptr(), (n, 1), cb.data_ptr(), (n, 1))
            names.append(dev.gemm_plan(desc)[2] + " bf16 A B")
            for _ in range(5):
                dev.gemm(desc)
            torch.cuda.synchronize()
            print(json.dumps({"probe": names}))
        elif args.probe == "f32-forms":
            del a, b, c
            a, b, c = (torch.randn(n, n, device="cuda", dtype=torch.float32) for _ in range(3))
            names = []
            for bstr in ((1, n), (n, 1)):
                probe = dev.gemm_desc("f32", n, n, n, a.data_ptr(), (n, 1), b.data_ptr(), bstr, c.data_ptr(), (n, 1), kernel=KERNEL_MFMA)
                by_name = {}
                for v in range(1, dev.mfma_variant_count("f32") + 1):
                    probe.variant = v
                    try:
                        by_name[dev.gemm_plan(probe)[2]] = v
                    except Exception:   # a variant that does not take this product
                        pass
                for v in (by_name["mfma32_256x256x32_w2x4"], by_name["mfma32_dma_256x256x32_w2x4"]):   # the register-staged 256x256 tile, the LDS-DMA form of it
                    desc = dev.gemm_desc("f32", n, n, n, a.data_ptr(), (n, 1), b.data_ptr(), bstr, c.data_ptr(), (n, 1),
                                         kernel=KERNEL_MFMA, variant=v, no_split_k=True)
                    names.append(dev.gemm_plan(desc)[2])
                    for _ in range(3):
                        dev.gemm(desc)
                    torch.cuda.synchronize()
            print(json.dumps({"probe": names}))
        elif args.probe == "rows":
            del a, b, c
            src = torch.ones(256 << 20, dtype=torch.uint8, device="cuda")
            dst = torch.empty_like(src)
            for _ in range(3):
                dst.copy_(src)
            torch.cuda.synchronize()
            del src, dst
            Bq, H, S, D = 8, 16, 1024, 64
            sSD, sSS = (H * S * D, S * D), (H * S * S, S * S)
            q, k, v, d_o = ((torch.randn(Bq, H, S, D, device="cuda")).half() for _ in range(4))
            sc = torch.zeros(Bq, H, S, S, device="cuda", dtype=torch.float16)
            gp, gs = torch.zeros_like(sc), torch.zeros_like(sc)
            P = lambda t: t.data_ptr()
            vw = lambda t: View(t.view(torch.uint8).reshape(-1), "f16", tuple(t.shape), tuple(t.stride()))
            scores = dev.gemm_desc("f16", S, D, S, P(q), (D, 1), P(k), (1, D), P(sc), (S, 1), batch=(Bq, H), a_batch=sSD, b_batch=sSD, c_batch=sSS)
            dp = dev.gemm_desc("f16", S, D, S, P(d_o), (D, 1), P(v), (1, D), P(gp), (S, 1), accumulate=True, batch=(Bq, H),
                               a_batch=sSD, b_batch=sSD, c_batch=sSS)
            n_ = 16384
            W, xv, yv = torch.randn(n_, n_, device="cuda").half(), torch.randn(n_, device="cuda").half(), torch.zeros(n_, device="cuda").half()
            gv = dev.gemm_desc("f16", 1, n_, n_, P(xv), (n_, 1), P(W), (n_, 1), P(yv), (n_, 1))
            r1 = dev.gemm_desc("f16", n_, 1, n_, P(xv), (1, 1), P(yv), (n_, 1), P(W), (n_, 1), accumulate=True)  # W += x (x) y: the gradient of gv
            # thin contractions: a rank-16 factor applied to 8192 rows, and attention scores with a head dimension of 32
            ta, tb = torch.randn(8192, 16, device="cuda").half(), torch.randn(16, 4096, device="cuda").half()
            tc = torch.zeros(8192, 4096, device="cuda", dtype=torch.float16)
            thin = dev.gemm_desc("f16", 8192, 16, 4096, P(ta), (16, 1), P(tb), (4096, 1), P(tc), (4096, 1))
            q32, k32 = ((torch.randn(Bq, H, S, 32, device="cuda")).half() for _ in range(2))
            s32 = (H * S * 32, S * 32)
            thin_scores = dev.gemm_desc("f16", S, 32, S, P(q32), (32, 1), P(k32), (1, 32), P(gs), (S, 1), batch=(Bq, H), a_batch=s32,
                                        b_batch=s32, c_batch=sSS)
            names = []
            for desc in (scores, dp, gv, r1, thin, thin_scores):
                names.append(dev.gemm_plan(desc)[2])
                for _ in range(3):
                    dev.gemm(desc)
                torch.cuda.synchronize()
            for _ in range(3):
                prob = dev.softmax_forward(vw(sc), 0.125)
                torch.cuda.synchronize()
            for _ in range(3):
                dev.softmax_backward(prob, vw(gs), vw(gp), 0.125)
                torch.cuda.synchronize()
            print(json.dumps({"probe": ["3 x 256 MiB copy"] + names + ["softmax_forward", "softmax_backward"]}))
        else:
            names = []
            for v in range(1, dev.mfma_variant_count("f16") + 1):
                desc = dev.gemm_desc("f16", n, n, n, a.data_ptr(), (n, 1), b.data_ptr(), (n, 1), c.data_ptr(), (n, 1),
                                     kernel=KERNEL_MFMA, variant=v, no_split_k=True)
                names.append(dev.gemm_plan(desc)[2])
                for _ in range(3):
                    dev.gemm(desc)
                torch.cuda.synchronize()
            print(json.dumps({"probe": names}))
        return
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32, "f64": torch.float64}
    esz = {"f16": 2, "bf16": 2, "f32": 4, "f64": 8}
    only = set(filter(None, args.only.split(",")))
    rows = []

    def want(group):
        return not only or group in only

    def rnd(shape, dtype, scale=1.0):
        return (torch.randn(*shape, device="cuda") * scale).to(tdt[dtype])

    def zeros(shape, dtype):
        return torch.zeros(*shape, device="cuda", dtype=tdt[dtype])

    def view(t, dtype):
        return View(t.view(torch.uint8).reshape(-1), dtype, tuple(t.shape), tuple(t.stride()))

    def report(group, name, flop, nbytes, ms, kernel, rot_ms=None, sets=0):
        row = {"group": group, "case": name, "kernel": kernel, "us": round(ms * 1e3, 2),
               "tflops": round(flop / ms / 1e9, 1) if flop else None,
               "gbps": round(nbytes / ms / 1e6, 1) if nbytes else None}
        tail = ""
        if rot_ms:   # the same case over `sets` disjoint buffer sets taken in turn: no launch finds its operands cached
            row.update({"sets": sets, "us_rotating": round(rot_ms * 1e3, 2),
                        "tflops_rotating": round(flop / rot_ms / 1e9, 1) if flop else None,
                        "gbps_rotating": round(nbytes / rot_ms / 1e6, 1) if nbytes else None})
            tail = f"  | {sets:3d} sets {row['us_rotating']:9.1f} us " + (
                f"{row['gbps_rotating']} GB/s" if nbytes else f"{row['tflops_rotating']} TFLOP/s")
        rows.append(row)
        print(f"{group:5s} {name:44s} {kernel:40s} {row['us']:9.1f} us "
              f"{(str(row['tflops']) + ' TFLOP/s') if flop else '':>16s} {(str(row['gbps']) + ' GB/s') if nbytes else '':>14s}{tail}",
              flush=True)

    def nsets(bufs):
        """Buffer sets that put more than the last-level cache (256 MB) in flight: at least 4, at most 512."""
        foot = sum(t.numel() * t.element_size() for t in bufs)
        return int(min(512, max(4, -(-ROTATE_BYTES // max(foot, 1)))))

    def gemm(group, name, desc, flop, nbytes, iters=None, bufs=None):
        """`bufs`: the tensors the descriptor points into; given, the case is also timed over rotating copies of them."""
        iters = iters or max(args.iters, 100)
        # 20 warm-up launches: a case of a few launches inherits the clock the case before it left behind (the same 60 us
        # product measured 60 or 68 us depending on what ran before it with 5 + 30 launches)
        ms = dev.gemm_time(desc, 20, iters)
        rot_ms, n = None, 0
        if bufs and not args.no_rotate:
            n = nsets(bufs)
            descs, keep = [desc], []
            for _ in range(n - 1):
                d = GemmDesc.from_buffer_copy(desc)
                copies = [t.clone() for t in bufs]
                keep.append(copies)
                for field in ("a", "b", "c", "bias"):
                    ptr = getattr(desc, field)
                    for t, cp in zip(bufs, copies):
                        if ptr is not None and t.data_ptr() <= ptr < t.data_ptr() + t.numel() * t.element_size():
                            setattr(d, field, cp.data_ptr() + (ptr - t.data_ptr()))
                descs.append(d)
            rot_ms = dev.gemm_time_rotating(descs, n, max(iters, 2 * n))
            del keep
        report(group, name, flop, nbytes, ms, dev.gemm_plan(desc)[2], rot_ms, n)

    def loop_ms(call, iters):
        for i in range(5):
            call(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(iters):
            call(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters

    def timed(group, name, fn, flop, nbytes, kernel, sets=None):
        """`sets`: the same call on disjoint buffers, one callable per set; results are held for one turn of the
        rotation so that the outputs an op allocates are disjoint too."""
        ms = loop_ms(lambda i: fn(), args.iters)
        rot_ms, n = None, 0
        if sets and not args.no_rotate:
            n = len(sets)
            hold = [None] * n

            def call(i):
                hold[i % n] = sets[i % n]()
            rot_ms = loop_ms(call, max(args.iters, 2 * n))
            del hold
        report(group, name, flop, nbytes, ms, kernel, rot_ms, n)

    def copies(n, *tensors):
        """n sets of the given tensors: the originals first, then n - 1 clones of each."""
        return [tensors] + [tuple(t.clone() for t in tensors) for _ in range(n - 1)]

    P = lambda t: t.data_ptr()

    # ---- config 1: Linear 512 -> 256 on 64 rows, f32 (latency-bound) ------------------------------------------
    if want("c1"):
        # the configuration itself is f32; the same three products in the other element types follow it
        for dt, es in (("f32", 4), ("f16", 2), ("bf16", 2), ("f64", 8)):
            r, i, o = 64, 512, 256
            tag = "" if dt == "f32" else f" [{dt}]"
            x, w, go = rnd((r, i), dt), rnd((o, i), dt, 0.04), rnd((r, o), dt)
            y, gx, gw = zeros((r, o), dt), zeros((r, i), dt), zeros((o, i), dt)
            fl = 2 * r * i * o
            gemm("c1", "Linear fwd 64x512x256 NT" + tag, dev.gemm_desc(dt, r, i, o, P(x), (i, 1), P(w), (1, i), P(y), (o, 1)),
                 fl, es * (r * i + i * o + r * o), 200, bufs=(x, w, y))
            gemm("c1", "dX 64x256x512 NN acc" + tag, dev.gemm_desc(dt, r, o, i, P(go), (o, 1), P(w), (i, 1), P(gx), (i, 1), accumulate=True),
                 fl, es * (r * o + i * o + 2 * r * i), 200, bufs=(go, w, gx))
            gemm("c1", "dW 512x64x256 TN col-major C acc" + tag,
                 dev.gemm_desc(dt, i, r, o, P(x), (1, i), P(go), (o, 1), P(gw), (1, i), accumulate=True),
                 fl, es * (r * o + r * i + 2 * i * o), 200, bufs=(x, go, gw))

    # ---- config 3: [32,512,1024] x [1024,1024], f16, broadcast rhs ---------------------------------------------
    if want("c3"):
        dt, (B, M, K, N), es = "f16", (32, 512, 1024, 1024), 2
        lhs, rhs, go = rnd((B, M, K), dt), rnd((K, N), dt, 1 / 32), rnd((B, M, N), dt)
        out, gl, gr = zeros((B, M, N), dt), zeros((B, M, K), dt), zeros((K, N), dt)
        fl = 2 * B * M * K * N
        gemm("c3", "fwd 16384x1024x1024 NN", dev.gemm_desc(dt, B * M, K, N, P(lhs), (K, 1), P(rhs), (N, 1), P(out), (N, 1)),
             fl, es * (B * M * K + K * N + B * M * N))
        gemm("c3", "fwd, rhs = Linear weight view NT",
             dev.gemm_desc(dt, B * M, K, N, P(lhs), (K, 1), P(rhs), (1, K), P(out), (N, 1)), fl, es * (B * M * K + K * N + B * M * N))
        gemm("c3", "dX 16384x1024x1024 NT acc",
             dev.gemm_desc(dt, B * M, N, K, P(go), (N, 1), P(rhs), (1, N), P(gl), (K, 1), accumulate=True),
             fl, es * (B * M * N + K * N + 2 * B * M * K))
        gemm("c3", "dW 1024x16384x1024 TN acc",
             dev.gemm_desc(dt, K, B * M, N, P(lhs), (1, K), P(go), (N, 1), P(gr), (N, 1), accumulate=True),
             fl, es * (B * M * K + B * M * N + 2 * K * N))
        lv, rv, gov, glv, grv = (view(t, dt) for t in (lhs, rhs, go, gl, gr))
        timed("c3", "MatMatBr forward (trait call, allocates out)", lambda: dev.forward(lv, rv), fl, 0, "br_forward")
        timed("c3", "MatMatBr backward (trait call, dX + dW)", lambda: dev.backward(lv, glv, rv, grv, gov), 2 * fl, 0, "br_backward")
        del lhs, rhs, go, out, gl, gr

    # ---- config 4: attention-shaped Rank-4, f16 -----------------------------------------------------------------
    if want("c4"):
        dt, (Bq, H, S, D), es = "f16", (8, 16, 1024, 64), 2
        q, k, v, d_o = (rnd((Bq, H, S, D), dt) for _ in range(4))
        sc = zeros((Bq, H, S, S), dt)
        p = torch.softmax(torch.randn(Bq, H, S, S, device="cuda"), -1).to(tdt[dt])
        o, gp, gv, gq, gk = zeros((Bq, H, S, D), dt), zeros((Bq, H, S, S), dt), zeros((Bq, H, S, D), dt), zeros((Bq, H, S, D), dt), zeros((Bq, H, S, D), dt)
        nb = Bq * H
        sSD, sSS = (H * S * D, S * D), (H * S * S, S * S)
        fl = 2 * nb * S * S * D

        def d4(m, kk, n, a, astr, ab, b, bstr, bb, c, cstr, cb, acc):
            return dev.gemm_desc(dt, m, kk, n, P(a), astr, P(b), bstr, P(c), cstr, accumulate=acc, batch=(Bq, H),
                                 a_batch=ab, b_batch=bb, c_batch=cb)

        gemm("c4", "scores Q.K^T 1024x64x1024 NT", d4(S, D, S, q, (D, 1), sSD, k, (1, D), sSD, sc, (S, 1), sSS, False),
             fl, es * nb * (2 * S * D + S * S), bufs=(q, k, sc))
        gemm("c4", "out P.V 1024x1024x64 NN", d4(S, S, D, p, (S, 1), sSS, v, (D, 1), sSD, o, (D, 1), sSD, False),
             fl, es * nb * (S * S + 2 * S * D), bufs=(p, v, o))
        gemm("c4", "dP dO.V^T NT acc", d4(S, D, S, d_o, (D, 1), sSD, v, (1, D), sSD, gp, (S, 1), sSS, True),
             fl, es * nb * (2 * S * D + 2 * S * S), bufs=(d_o, v, gp))
        dp_desc = d4(S, D, S, d_o, (D, 1), sSD, v, (1, D), sSD, gp, (S, 1), sSS, True)

        def dp_fresh():   # the same accumulation into a gradient that is only DECLARED zero: stored, not read
            dev.zero_deferred(P(gp), gp.numel() * es)
            dev.gemm(dp_desc)
        timed("c4", "dP acc into a deferred-zero gradient", dp_fresh, fl, es * nb * (2 * S * D + S * S), "gemm, beta = 0 by declaration")
        gemm("c4", "dV P^T.dO TN acc", d4(S, S, D, p, (1, S), sSS, d_o, (D, 1), sSD, gv, (D, 1), sSD, True),
             fl, es * nb * (S * S + 3 * S * D), bufs=(p, d_o, gv))
        gemm("c4", "dQ dS.K NN acc", d4(S, S, D, gp, (S, 1), sSS, k, (D, 1), sSD, gq, (D, 1), sSD, True),
             fl, es * nb * (S * S + 3 * S * D), bufs=(gp, k, gq))
        gemm("c4", "dK^T Q^T.dS col-major C acc", d4(D, S, S, q, (1, D), sSD, gp, (S, 1), sSS, gk, (1, D), sSD, True),
             fl, es * nb * (S * S + 3 * S * D), bufs=(q, gp, gk))
        if want("glue"):
            scv, pv, gpv, ov = view(sc, dt), view(p, dt), view(gp, dt), view(o, dt)
            mat = nb * S * S * es
            vw = lambda t: view(t, dt)
            timed("glue", "softmax fwd (8,16,1024,1024) f16, scale folded", lambda: dev.softmax_forward(scv, 0.125), 0, 2 * mat, "softmax_forward",
                  sets=[(lambda a=vw(t): dev.softmax_forward(a, 0.125)) for (t,) in copies(4, sc)])
            gs = zeros((Bq, H, S, S), dt)
            gsv = view(gs, dt)
            timed("glue", "softmax bwd (8,16,1024,1024) f16", lambda: dev.softmax_backward(pv, gsv, gpv, 0.125), 0, 4 * mat, "softmax_backward",
                  sets=[(lambda a=vw(t0), b=vw(t1), c=vw(t2): dev.softmax_backward(a, b, c, 0.125)) for t0, t1, t2 in copies(4, p, gs, gp)])
            tok = nb * S * D * es
            timed("glue", "reshape copy (B,H,S,D)->(B,S,H*D) f16", lambda: dev.reshape_forward(ov.permute(0, 2, 1, 3), (Bq, S, H * D)), 0, 2 * tok, "reshape_forward",
                  sets=[(lambda a=vw(t): dev.reshape_forward(a.permute(0, 2, 1, 3), (Bq, S, H * D))) for (t,) in copies(12, o)])
            g_t, g_o = rnd((Bq, S, H * D), dt), zeros((Bq, H, S, D), dt)
            gt, gov = view(g_t, dt), view(g_o, dt)
            timed("glue", "reshape backward (scatter-add) f16", lambda: dev.reshape_backward(ov.permute(0, 2, 1, 3), gov, gt), 0, 3 * tok, "reshape_backward",
                  sets=[(lambda a=vw(t0), b=vw(t1), c=vw(t2): dev.reshape_backward(a.permute(0, 2, 1, 3), b, c)) for t0, t1, t2 in copies(8, o, g_o, g_t)])
            del gs, g_t, g_o
        del sc, p, gp

    # ---- config 5: the encoder block's Linears, bf16, 8192 tokens ----------------------------------------------
    if want("c5"):
        dt, T = "bf16", 8192
        for name, kin, nout in (("qkv / out proj", 1024, 1024), ("ff1", 1024, 4096), ("ff2", 4096, 1024)):
            x, w, go = rnd((T, kin), dt), rnd((nout, kin), dt, 0.02), rnd((T, nout), dt)
            y, gx, gw = zeros((T, nout), dt), zeros((T, kin), dt), zeros((nout, kin), dt)
            fl = 2 * T * kin * nout
            gemm("c5", f"{name} fwd {T}x{kin}x{nout} NT", dev.gemm_desc(dt, T, kin, nout, P(x), (kin, 1), P(w), (1, kin), P(y), (nout, 1)), fl, 0)
            bvec = rnd((nout,), dt)
            gemm("c5", f"{name} fwd with fused bias (Linear)",
                 dev.gemm_desc(dt, T, kin, nout, P(x), (kin, 1), P(w), (1, kin), P(y), (nout, 1), bias=P(bvec)), fl, 0)
            gemm("c5", f"{name} dX NN acc", dev.gemm_desc(dt, T, nout, kin, P(go), (nout, 1), P(w), (kin, 1), P(gx), (kin, 1), accumulate=True), fl, 0)
            gemm("c5", f"{name} dW TN col-major C acc",
                 dev.gemm_desc(dt, kin, T, nout, P(x), (1, kin), P(go), (nout, 1), P(gw), (1, kin), accumulate=True), fl, 0)
            if want("glue"):
                gb = zeros((nout,), dt)
                gov, gbv = view(go, dt), view(gb, dt)
                timed("glue", f"bias backward {T}x{nout} bf16", lambda: dev.bias_backward(gov, gbv), 0, T * nout * 2, "bias_backward",
                      sets=[(lambda a=view(t0, dt), b=view(t1, dt): dev.bias_backward(a, b)) for t0, t1 in copies(nsets((go,)), go, gb)])

        # the block's attention products: heads interleaved in the token rows (batch-2 stride 64 < row stride 1024),
        # as MultiHeadAttention's reshape + permute hands them over (multi_head_attention.rs:105-146)
        Bq, H, S, D, es = 16, 16, 512, 64, 2
        nb = Bq * H
        q, k, v, d_o = (rnd((Bq, S, H * D), dt) for _ in range(4))
        sc, p_, gp = zeros((Bq, H, S, S), dt), rnd((Bq, H, S, S), dt, 0.05), zeros((Bq, H, S, S), dt)
        o, gv = zeros((Bq, H, S, D), dt), zeros((Bq, S, H * D), dt)
        tok, sSS, sSD = (S * H * D, D), (H * S * S, S * S), (H * S * D, S * D)
        fl = 2 * nb * S * S * D

        def d5(m, kk, n, a, astr, ab, b, bstr, bb, c, cstr, cb, acc):
            return dev.gemm_desc(dt, m, kk, n, P(a), astr, P(b), bstr, P(c), cstr, accumulate=acc, batch=(Bq, H),
                                 a_batch=ab, b_batch=bb, c_batch=cb)

        gemm("c5", "attn scores Q.K^T 512x64x512 interleaved", d5(S, D, S, q, (H * D, 1), tok, k, (1, H * D), tok, sc, (S, 1), sSS, False),
             fl, es * nb * (2 * S * D + S * S), bufs=(q, k, sc))
        gemm("c5", "attn out P.V 512x512x64 interleaved V", d5(S, S, D, p_, (S, 1), sSS, v, (H * D, 1), tok, o, (D, 1), sSD, False),
             fl, es * nb * (S * S + 2 * S * D), bufs=(p_, v, o))
        gemm("c5", "attn dP dO.V^T acc", d5(S, D, S, d_o, (D, 1), sSD, v, (1, H * D), tok, gp, (S, 1), sSS, True),
             fl, es * nb * (2 * S * D + 2 * S * S), bufs=(d_o, v, gp))
        gemm("c5", "attn dV P^T.dO acc, interleaved rows", d5(S, S, D, p_, (1, S), sSS, d_o, (D, 1), sSD, gv, (H * D, 1), tok, True),
             fl, es * nb * (S * S + 3 * S * D), bufs=(p_, d_o, gv))
        if want("glue"):
            vw = lambda t: view(t, dt)
            mat = nb * S * S * es
            timed("glue", "softmax fwd (16,16,512,512) bf16, scale folded", lambda: dev.softmax_forward(vw(sc), 0.125), 0, 2 * mat, "softmax_forward",
                  sets=[(lambda a=vw(t): dev.softmax_forward(a, 0.125)) for (t,) in copies(4, sc)])
            gs = zeros((Bq, H, S, S), dt)
            timed("glue", "softmax bwd (16,16,512,512) bf16", lambda: dev.softmax_backward(vw(p_), vw(gs), vw(gp), 0.125), 0, 4 * mat, "softmax_backward",
                  sets=[(lambda a=vw(t0), b=vw(t1), c=vw(t2): dev.softmax_backward(a, b, c, 0.125)) for t0, t1, t2 in copies(4, p_, gs, gp)])
            del gs
        del sc, p_, gp

    # ---- zero fill of gradient storage (Storage::try_alloc_len): HBM write roofline -----------------------------
    if want("fill"):
        import ctypes

        for mb in (2, 16, 64, 256):   # config 5's weight, activation, ff activation and probability gradients
            nbytes = mb << 20
            buf = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
            ptr = ctypes.c_void_p(buf.data_ptr())
            n = nsets((buf,))
            more = [torch.empty(nbytes, dtype=torch.uint8, device="cuda") for _ in range(n - 1)]
            ptrs = [ptr] + [ctypes.c_void_p(t.data_ptr()) for t in more]
            timed("fill", f"zero fill {mb} MiB (dfdx_rocm_memset_zero)",
                  lambda: dev._check(dev.lib.dfdx_rocm_memset_zero(dev.ctx, ptr, ctypes.c_size_t(nbytes))), 0, nbytes, "zero_fill_kernel",
                  sets=[(lambda q=q: dev._check(dev.lib.dfdx_rocm_memset_zero(dev.ctx, q, ctypes.c_size_t(nbytes)))) for q in ptrs])
            timed("fill", f"zero fill {mb} MiB (torch zero_, for comparison)", lambda: buf.zero_(), 0, nbytes, "torch fill",
                  sets=[(lambda t=t: t.zero_()) for t in [buf] + more])
            del more
            del buf

    # ---- the vendor library on the same shapes (torch.matmul = hipBLASLt / rocBLAS), for orientation only ---------
    if "torch" in only:   # not part of the default run: a cross-check, never a code path of the library
        def pair(name, dt, fn_ours_desc, fn_torch, flop):
            gemm("torch", name + " (this library)", fn_ours_desc, flop, 0)
            timed("torch", name + " (torch.matmul)", fn_torch, flop, 0, "vendor library")

        n = 4096
        for dt in ("f16", "bf16", "f32"):
            a, b, c = rnd((n, n), dt), rnd((n, n), dt), zeros((n, n), dt)
            pair(f"4096^3 {dt} A.B", dt, dev.gemm_desc(dt, n, n, n, P(a), (n, 1), P(b), (n, 1), P(c), (n, 1)),
                 lambda: torch.matmul(a, b, out=c), 2 * n ** 3)
        dt = "f16"
        x, w, go = rnd((16384, 1024), dt), rnd((1024, 1024), dt, 0.03), rnd((16384, 1024), dt)
        y, gw = zeros((16384, 1024), dt), zeros((1024, 1024), dt)
        pair("c3 fwd 16384x1024x1024 NN f16", dt, dev.gemm_desc(dt, 16384, 1024, 1024, P(x), (1024, 1), P(w), (1024, 1), P(y), (1024, 1)),
             lambda: torch.matmul(x, w, out=y), 2 * 16384 * 1024 * 1024)
        pair("c3 dW 1024x16384x1024 TN f16 (beta = 1 here, overwrite in torch)", dt,
             dev.gemm_desc(dt, 1024, 16384, 1024, P(x), (1, 1024), P(go), (1024, 1), P(gw), (1024, 1), accumulate=True),
             lambda: torch.matmul(x.t(), go, out=gw), 2 * 16384 * 1024 * 1024)
        dt, T = "bf16", 8192
        x, w, go = rnd((T, 1024), dt), rnd((4096, 1024), dt, 0.02), rnd((T, 4096), dt)
        y, gw = zeros((T, 4096), dt), zeros((4096, 1024), dt)
        pair("c5 ff1 fwd 8192x1024x4096 NT bf16", dt, dev.gemm_desc(dt, T, 1024, 4096, P(x), (1024, 1), P(w), (1, 1024), P(y), (4096, 1)),
             lambda: torch.matmul(x, w.t(), out=y), 2 * T * 1024 * 4096)
        pair("c5 ff1 dW TN col-major C bf16 (beta = 1 here, overwrite in torch)", dt,
             dev.gemm_desc(dt, 1024, T, 4096, P(x), (1, 1024), P(go), (4096, 1), P(gw), (1, 1024), accumulate=True),
             lambda: torch.matmul(go.t(), x, out=gw), 2 * T * 1024 * 4096)
        dt, nb, S, D = "f16", 128, 1024, 64
        q, k_, pm = rnd((nb, S, D), dt), rnd((nb, S, D), dt), rnd((nb, S, S), dt, 0.03)
        sc, o = zeros((nb, S, S), dt), zeros((nb, S, D), dt)
        pair("c4 scores Q.K^T 128 x 1024x64x1024 f16", dt,
             dev.gemm_desc(dt, S, D, S, P(q), (D, 1), P(k_), (1, D), P(sc), (S, 1), batch=(nb, 1), a_batch=(S * D, 0), b_batch=(S * D, 0), c_batch=(S * S, 0)),
             lambda: torch.bmm(q, k_.transpose(1, 2), out=sc), 2 * nb * S * S * D)
        pair("c4 out P.V 128 x 1024x1024x64 f16", dt,
             dev.gemm_desc(dt, S, S, D, P(pm), (S, 1), P(q), (D, 1), P(o), (D, 1), batch=(nb, 1), a_batch=(S * S, 0), b_batch=(S * D, 0), c_batch=(S * D, 0)),
             lambda: torch.bmm(pm, q, out=o), 2 * nb * S * S * D)

    # ---- vec.mat / mat.vec: HBM roofline ------------------------------------------------------------------------
    if want("gemv"):
        for dt in ("f16", "f32"):
            es = esz[dt]
            for n_ in (4096, 16384):
                W, xv, yv = rnd((n_, n_), dt), rnd((n_,), dt), zeros((n_,), dt)
                gemm("gemv", f"vec.mat {dt} (1,{n_})x({n_},{n_})", dev.gemm_desc(dt, 1, n_, n_, P(xv), (n_, 1), P(W), (n_, 1), P(yv), (n_, 1)), 2 * n_ * n_, es * n_ * n_, 100, bufs=(W, xv, yv))
                gemm("gemv", f"vec.mat {dt}, Linear weight view", dev.gemm_desc(dt, 1, n_, n_, P(xv), (n_, 1), P(W), (1, n_), P(yv), (n_, 1)), 2 * n_ * n_, es * n_ * n_, 100, bufs=(W, xv, yv))
                gemm("gemv", f"mat.vec {dt} ({n_},{n_})x({n_},)", dev.gemm_desc(dt, n_, n_, 1, P(W), (n_, 1), P(xv), (1, 1), P(yv), (1, 1)), 2 * n_ * n_, es * n_ * n_, 100, bufs=(W, xv, yv))
                # the weight gradient of the same vec.mat: the rank-1 update grad_W += x^T (x) grad_y (k = 1), C read and written
                gemm("gemv", f"rank-1 update {dt} ({n_},1)x(1,{n_}) acc", dev.gemm_desc(dt, n_, 1, n_, P(xv), (1, 1), P(yv), (n_, 1), P(W), (n_, 1), accumulate=True),
                     2 * n_ * n_, 2 * es * n_ * n_, 100, bufs=(W, xv, yv))
                del W

    # ---- shapes outside the five configurations: few rows or columns, thin contractions, rank-1 updates, mid-size --------
    if "shapes" in only:   # on request: which kernel the planner gives each shape class, and what it costs
        cases = [  # (m, k, n, layout of A and B: n = stored as indexed, t = stored transposed)
            (64, 512, 256, "nt"), (256, 256, 256, "nt"), (100, 300, 200, "nn"), (512, 512, 512, "nt"), (1000, 1000, 1000, "nn"), (2048, 2048, 2048, "nt"),
            (4096, 1, 4096, "nn"), (4095, 1, 4097, "nn"), (8192, 4, 1024, "nt"), (65536, 8, 256, "nt"), (8192, 10, 1024, "nn"), (4096, 16, 4096, "nn"),
            (4, 4096, 4096, "nt"), (4, 4096, 4096, "nn"), (8, 1024, 50264, "nt"), (16, 4096, 4096, "nt"), (32, 8192, 8192, "nt"),
            (65536, 512, 2, "nt"), (8192, 1024, 10, "nt"), (10, 8192, 1024, "tn"), (1024, 8192, 10, "tn"),
        ]
        for dt in ("f16", "f32", "f64"):
            es = esz[dt]
            for m, k, n, lay in cases:
                if dt == "f64" and m * k * n > 2 ** 31:
                    continue
                a = rnd((k, m) if lay[0] == "t" else (m, k), dt)
                b = rnd((n, k) if lay[1] == "t" else (k, n), dt)
                c = zeros((m, n), dt)
                desc = dev.gemm_desc(dt, m, k, n, P(a), (1, m) if lay[0] == "t" else (k, 1), P(b), (1, k) if lay[1] == "t" else (n, 1), P(c), (n, 1))
                gemm("shape", f"{dt} {m}x{k}x{n} {lay}", desc, 2 * m * k * n, es * (m * k + k * n + m * n), 100)
                del a, b, c

    # ---- planner regression check: the automatic pick against every forced candidate ---------------------------------
    flagged = []
    if "plancheck" in only or "fewrows" in only:
        from dfdx_amd.rocm import KERNEL_GEMV, KERNEL_MFMA, RocmError

        # (dtype, m, k, n, layout of A and B (n = stored as indexed, t = transposed), accumulate, batch)
        T = 8192
        pc_cases = [("f16", 4096, 4096, 4096, "nn", False, 1), ("f16", 4096, 4096, 4096, "tn", False, 1), ("f16", 4096, 4096, 4096, "nt", False, 1),
                    ("f32", 4096, 4096, 4096, "nn", False, 1), ("f32", 64, 512, 256, "nt", False, 1), ("f32", 64, 256, 512, "nn", True, 1),
                    ("f32", 512, 64, 256, "tn", True, 1),
                    ("f16", 16384, 1024, 1024, "nn", False, 1), ("f16", 16384, 1024, 1024, "nt", True, 1), ("f16", 1024, 16384, 1024, "tn", True, 1),
                    ("f16", 1024, 64, 1024, "nt", False, 128), ("f16", 1024, 1024, 64, "nn", False, 128), ("f16", 1024, 1024, 64, "tn", True, 128),
                    ("bf16", T, 1024, 1024, "nt", False, 1), ("bf16", T, 1024, 4096, "nt", False, 1), ("bf16", T, 4096, 1024, "nt", False, 1),
                    ("bf16", T, 1024, 1024, "nn", True, 1), ("bf16", T, 4096, 1024, "nn", True, 1), ("bf16", T, 1024, 4096, "nn", True, 1),
                    ("bf16", 1024, T, 1024, "tn", True, 1), ("bf16", 4096, T, 1024, "tn", True, 1), ("bf16", 1024, T, 4096, "tn", True, 1),
                    ("bf16", 512, 64, 512, "nt", False, 256), ("bf16", 512, 512, 64, "nn", False, 256),
                    ("f16", 2048, 2048, 2048, "nn", False, 1), ("f16", 1024, 1024, 1024, "nn", False, 1), ("f16", 512, 512, 512, "nt", False, 1),
                    ("f16", 256, 256, 256, "nt", False, 1), ("f16", 512, 4096, 512, "nn", False, 1), ("f16", 8192, 1024, 8192, "nt", False, 1),
                    ("f16", 16, 4096, 4096, "nt", False, 1), ("f16", 32, 8192, 8192, "nt", False, 1), ("f16", 4, 4096, 4096, "nt", False, 1),
                    ("f32", 2048, 2048, 2048, "nn", False, 1), ("f32", 1024, 8192, 1024, "tn", True, 1), ("f32", 8192, 1024, 1024, "nt", False, 1),
                    ("f32", 512, 512, 512, "nn", False, 1), ("f32", 16, 4096, 4096, "nt", False, 1)]
        # a Linear layer on a handful of rows, both weight layouts: where the multi-vector kernel, the k-sliced small kernel and
        # the split tiles meet
        few_cases = [(dt, r, k, n, lay, False, 1) for dt in ("f16", "f32") for lay in ("nt", "nn") for r in (2, 4, 8, 16)
                     for k, n in ((1024, 1024), (2048, 2048), (4096, 4096), (8192, 8192), (4096, 16384), (16384, 4096), (8192, 1024), (1024, 8192))]

        def plancheck_run(cases, label):
            for dt, m, k, n, lay, acc, nb in cases:
                a = rnd((nb, k, m) if lay[0] == "t" else (nb, m, k), dt)
                b = rnd((nb, n, k) if lay[1] == "t" else (nb, k, n), dt, k ** -0.5)
                c = zeros((nb, m, n), dt)

                def pc_desc(kernel=0, variant=0, split=0):
                    return dev.gemm_desc(dt, m, k, n, P(a), (1, m) if lay[0] == "t" else (k, 1), P(b), (1, k) if lay[1] == "t" else (n, 1), P(c), (n, 1),
                                         accumulate=acc, batch=(nb, 1), a_batch=(m * k, 0), b_batch=(k * n, 0), c_batch=(m * n, 0),
                                         kernel=kernel, variant=variant, split_k=split, no_split_k=(split == 1))

                def pc_time(desc, iters=20):
                    try:
                        name = dev.gemm_plan(desc)[2]
                        return min(dev.gemm_time(desc, 3, iters), dev.gemm_time(desc, 1, iters)), name
                    except RocmError:
                        return None, None

                auto_ms, auto_name = pc_time(pc_desc())
                cands = {}
                for v in range(1, dev.mfma_variant_count(dt) + 1):
                    for split in (1, 2, 4, 8, 16):
                        if split > 1 and (nb > 1 or k < 64 * 4 * split):
                            continue
                        ms, name = pc_time(pc_desc(KERNEL_MFMA, v, split), 10)
                        if ms and (name not in cands or ms < cands[name]):
                            cands[name] = ms
                ms, name = pc_time(pc_desc(KERNEL_GEMV), 10)
                if ms:
                    cands[name] = ms
                best_name = min(cands, key=cands.get)
                auto_ms = min(auto_ms, pc_time(pc_desc())[0])   # once more after the sweep: clocks drift over a run
                # the same plan under both names is the same launch: what separates the two timings is noise
                slack = 0.0 if best_name == auto_name else auto_ms / cands[best_name] - 1.0
                flag = slack > args.plancheck_slack
                tag = f"{dt} {'b' + str(nb) + ' ' if nb > 1 else ''}{m}x{k}x{n} {lay}{' acc' if acc else ''}"
                rows.append({"group": label, "case": tag, "kernel": auto_name, "us": round(auto_ms * 1e3, 2), "best": best_name,
                             "best_us": round(cands[best_name] * 1e3, 2), "candidates": len(cands), "off_best_pct": round(100 * slack, 1), "flagged": flag})
                print(f"{label[:5]:5s} {tag:34s} auto {auto_ms * 1e3:8.1f} us {auto_name:40s} best of {len(cands):3d} {cands[best_name] * 1e3:8.1f} us {best_name:40s} "
                      f"{100 * slack:+6.1f} %{'  <<<< FLAG' if flag else ''}", flush=True)
                if flag:
                    flagged.append(tag)
                del a, b, c
            mine = [r for r in rows if r["group"] == label]
            bad = [r["case"] for r in mine if r["flagged"]]
            print(f"{label}: {len(cases)} shapes, {len(bad)} flagged (pick more than {100 * args.plancheck_slack:.0f} % off the best forced candidate)"
                  + (": " + "; ".join(bad) if bad else ""), flush=True)

        if "plancheck" in only:
            plancheck_run(pc_cases, "plancheck")
        if "fewrows" in only:
            plancheck_run(few_cases, "fewrows")

    # ---- operands off the 16-byte grid: an LM head with 50257 outputs, a first-layer convolution -------------------
    if "edge" in only:   # on request: the scalar kernel's rows take milliseconds each
        from dfdx_amd.rocm import KERNEL_GENERIC
        for dt in ("f16", "f32"):
            M, K = 2048, 1024
            for N in (50257, 50264):
                x, W, y = rnd((M, K), dt), rnd((N, K), dt, 0.03), zeros((M, N), dt)
                go, gx, gw = rnd((M, N), dt), zeros((M, K), dt), zeros((N, K), dt)
                fl = 2.0 * M * K * N
                cases = (("LM head fwd x.W^T", (M, K, N, P(x), (K, 1), P(W), (1, K), P(y), (N, 1)), False),
                         ("LM head dX go.W", (M, N, K, P(go), (N, 1), P(W), (K, 1), P(gx), (K, 1)), True),
                         ("LM head dW go^T.x", (N, M, K, P(go), (1, N), P(x), (K, 1), P(gw), (K, 1)), True))
                for name, a, acc in cases:
                    gemm("edge", f"{name} {dt} N={N}", dev.gemm_desc(dt, *a, accumulate=acc), fl, 0, 10)
                    if N % 8:
                        gemm("edge", f"{name} {dt} N={N}, scalar kernel forced", dev.gemm_desc(dt, *a, accumulate=acc, kernel=KERNEL_GENERIC), fl, 0, 3)
                del x, W, y, go, gx, gw
        for dt in ("f16", "f32"):
            B, C, O, H, W_, K = 32, 3, 64, 224, 224, 3
            xv, wv = view(rnd((B, C, H, W_), dt), dt), view(rnd((O, C, K, K), dt, 0.2), dt)
            fl = 2.0 * B * O * C * K * K * H * W_
            timed("edge", f"conv2d fwd {dt} B{B} 3->64 224x224 k3 (C*K*K = 27)", lambda: dev.conv2d_forward(xv, wv, stride=1, padding=1), fl, 0, "conv2d_forward")

    # ---- config 5 end to end: one encoder block, every op on the device -----------------------------------------
    if want("block"):
        from dfdx_amd.encoder import EncoderBlock
        dt, (B, S, d, H, ff) = "bf16", (16, 512, 1024, 16, 4096)
        T = B * S
        shapes = {"wq": (d, d), "wk": (d, d), "wv": (d, d), "wo": (d, d), "w1": (ff, d), "w2": (d, ff),
                  "bq": (d,), "bk": (d,), "bv": (d,), "bo": (d,), "b1": (ff,), "b2": (d,)}
        params = {n: view(rnd(sh, dt, 0.02), dt) for n, sh in shapes.items()}
        for n in ("g1", "g2"):
            params[n] = view(torch.ones(d, device="cuda", dtype=tdt[dt]), dt)
        for n in ("be1", "be2"):
            params[n] = view(zeros((d,), dt), dt)
        blk = EncoderBlock(dev, dt, d, H, ff, params)
        xv, gv = view(rnd((B, S, d), dt), dt), view(rnd((B, S, d), dt, 1.0 / T), dt)
        D = d // H
        fwd_flop = 2.0 * T * d * d * 4 + 2 * 2.0 * T * d * ff + 2 * 2.0 * B * H * S * S * D
        ln_bytes = 2 * (2 * T * d * 2)
        timed("block", "encoder block forward (20 calls)", lambda: blk.forward(xv), fwd_flop, 0, "EncoderBlock.forward")
        _, saved = blk.forward(xv)
        timed("block", "encoder block backward (37 calls, gradient zeros deferred)", lambda: blk.backward(saved, gv), 2 * fwd_flop, 0, "EncoderBlock.backward")

        def step():
            _, sv = blk.forward(xv)
            blk.backward(sv, gv)
        timed("block", "encoder block forward + backward", step, 3 * fwd_flop, 0, "EncoderBlock")
        x_t, g_t = rnd((B, S, d), dt), rnd((B, S, d), dt, 1.0 / T)
        xs, gs_ = view(x_t, dt), view(g_t, dt)
        vw = lambda t: view(t, dt)
        g1, be1 = params["g1"], params["be1"]
        timed("glue", f"layer norm fwd ({T},{d}) {dt}", lambda: dev.layer_norm_forward(xs, g1, be1), 0, ln_bytes, "layer_norm_forward",
              sets=[(lambda a=vw(t): dev.layer_norm_forward(a, g1, be1)) for (t,) in copies(20, x_t)])
        gx_t, gg, gb = zeros((B, S, d), dt), view(zeros((d,), dt), dt), view(zeros((d,), dt), dt)
        gx = view(gx_t, dt)
        timed("glue", f"layer norm bwd ({T},{d}) {dt}", lambda: dev.layer_norm_backward(xs, g1, gx, gg, gb, gs_), 0, 2 * ln_bytes, "layer_norm_backward",
              sets=[(lambda a=vw(t0), b=vw(t1), c=vw(t2): dev.layer_norm_backward(a, g1, b, gg, gb, c)) for t0, t1, t2 in copies(8, x_t, gx_t, g_t)])
        f_t = rnd((B, S, ff), dt)
        f1 = view(f_t, dt)
        timed("glue", f"relu fwd ({T},{ff}) {dt}", lambda: dev.relu_forward(f1), 0, 2 * T * ff * 2, "relu_forward",
              sets=[(lambda a=vw(t): dev.relu_forward(a)) for (t,) in copies(6, f_t)])
        timed("glue", f"residual add fwd ({T},{d}) {dt}", lambda: dev.add_forward(xs, gs_), 0, 3 * T * d * 2, "add_forward",
              sets=[(lambda a=vw(t0), b=vw(t1): dev.add_forward(a, b)) for t0, t1 in copies(12, x_t, g_t)])
        del x_t, g_t, gx_t, f_t

    # ---- conv2d (unfold + batched GEMM) -------------------------------------------------------------------------
    if want("conv"):
        for dt, (B, C, O, H, W_, K, s, pad) in (("f16", (64, 64, 64, 56, 56, 3, 1, 1)), ("f16", (64, 128, 128, 28, 28, 3, 1, 1)),
                                                ("f16", (64, 256, 256, 14, 14, 3, 1, 1)), ("f16", (64, 512, 512, 7, 7, 3, 1, 1)),
                                                ("f16", (64, 256, 64, 56, 56, 1, 1, 0)),
                                                ("f32", (32, 64, 64, 56, 56, 3, 1, 1))):
            x, w = rnd((B, C, H, W_), dt), rnd((O, C, K, K), dt, 1 / 24)
            xv, wv = view(x, dt), view(w, dt)
            y = dev.conv2d_forward(xv, wv, stride=s, padding=pad)
            gov = view(rnd(y.shape, dt), dt)
            gxv, gwv = view(zeros((B, C, H, W_), dt), dt), view(zeros((O, C, K, K), dt), dt)
            fl = 2.0 * B * O * C * K * K * y.shape[2] * y.shape[3]
            tag = f"{dt} B{B} {C}->{O} {H}x{W_} k{K}"
            timed("conv", f"conv2d fwd {tag}", lambda: dev.conv2d_forward(xv, wv, stride=s, padding=pad), fl, 0, "conv2d_forward")
            timed("conv", f"conv2d bwd {tag}", lambda: dev.conv2d_backward(xv, gxv, wv, gwv, gov, stride=s, padding=pad), 2 * fl, 0, "conv2d_backward")

    # ---- conv2d outside the configurations' shapes (on request): strides, a first layer, depthwise, wide rows --------------
    if "convx" in only:
        # batch, chan_in, chan_out, h, w, kernel, stride, padding, groups
        for dt, (B, C, O, H, W_, K, s, pad, G) in (("f16", (64, 64, 128, 56, 56, 3, 2, 1, 1)), ("f16", (64, 128, 256, 28, 28, 3, 2, 1, 1)),
                                                   ("f16", (64, 256, 512, 14, 14, 3, 2, 1, 1)), ("f16", (64, 64, 128, 56, 56, 1, 2, 0, 1)),
                                                   ("f16", (64, 3, 64, 224, 224, 7, 2, 3, 1)), ("f16", (64, 3, 64, 32, 32, 3, 1, 1, 1)),
                                                   ("f32", (64, 3, 64, 32, 32, 3, 1, 1, 1)), ("f16", (64, 128, 128, 28, 28, 3, 1, 1, 128)),
                                                   ("f16", (32, 128, 128, 112, 112, 3, 1, 1, 1)), ("f16", (32, 64, 64, 224, 224, 3, 1, 1, 1)),
                                                   ("f32", (32, 512, 512, 7, 7, 3, 1, 1, 1)), ("f16", (64, 64, 64, 56, 56, 5, 1, 2, 1))):
            x, w = rnd((B, C, H, W_), dt), rnd((O, C // G, K, K), dt, 1 / 24)
            xv, wv = view(x, dt), view(w, dt)
            kw = dict(stride=s, padding=pad, groups=G)
            y = dev.conv2d_forward(xv, wv, **kw)
            gov = view(rnd(y.shape, dt), dt)
            gxv, gwv = view(zeros((B, C, H, W_), dt), dt), view(zeros((O, C // G, K, K), dt), dt)
            fl = 2.0 * B * O * (C // G) * K * K * y.shape[2] * y.shape[3]
            tag = f"{dt} B{B} {C}->{O} {H}x{W_} k{K} s{s}" + (f" groups {G}" if G > 1 else "")
            timed("convx", f"conv2d fwd {tag}", lambda: dev.conv2d_forward(xv, wv, **kw), fl, 0, "conv2d_forward")
            timed("convx", f"conv2d bwd {tag}", lambda: dev.conv2d_backward(xv, gxv, wv, gwv, gov, **kw), 2 * fl, 0, "conv2d_backward")
            del x, w, y

    # ---- softmax and LayerNorm on rows past what a wave keeps in registers (on request) --------------------------------
    if "longrows" in only:
        for dt in ("f16", "f32"):
            for R, Cc in ((4096, 5120), (8192, 4096), (64, 50257), (2048, 8192)):
                x_t, g_t = rnd((R, Cc), dt), rnd((R, Cc), dt)
                xs, gs_ = view(x_t, dt), view(g_t, dt)
                nbytes = R * Cc * esz[dt]
                p_ = dev.softmax_forward(xs)
                gx = view(zeros((R, Cc), dt), dt)
                timed("longrows", f"softmax fwd ({R},{Cc}) {dt}", lambda: dev.softmax_forward(xs), 0, 2 * nbytes, "softmax_forward")
                timed("longrows", f"softmax bwd ({R},{Cc}) {dt}", lambda: dev.softmax_backward(p_, gx, gs_), 0, 4 * nbytes, "softmax_backward")
                if Cc % 8 == 0:
                    g1, be1 = view(rnd((Cc,), dt), dt), view(rnd((Cc,), dt), dt)
                    gg, gb = view(zeros((Cc,), dt), dt), view(zeros((Cc,), dt), dt)
                    timed("longrows", f"layer norm fwd ({R},{Cc}) {dt}", lambda: dev.layer_norm_forward(xs, g1, be1), 0, 2 * nbytes, "layer_norm_forward")
                    timed("longrows", f"layer norm bwd ({R},{Cc}) {dt}", lambda: dev.layer_norm_backward(xs, g1, gx, gg, gb, gs_), 0, 4 * nbytes, "layer_norm_backward")
                del x_t, g_t, p_

    if args.json:
        with open(args.json, "w") as f:
            json.dump({"device": dev.device_info(), "rows": rows}, f, indent=1)
    if args.strict and flagged:
        sys.exit(1)


if __name__ == "__main__":
    main()
