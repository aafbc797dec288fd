#!/usr/bin/env python3
"""Benchmark of the fp32-in / fp16-MFMA / fp32-accumulate GEMM path on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input: one 8192^3 GEMM
(seeded N(0, 1/sqrt(K)) operands, resident in HBM before the timed region).  Prints ONE JSON
line.  `--workload` selects another configuration for profiling runs (the default is the one
the headline metric is quoted on)."""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS_FP16 = 2500.0      # MI355X dense fp16 MFMA
PEAK_HBM_GBPS = 8000.0         # MI355X HBM3E
PEAK_TFLOPS_FP32 = 157.3      # MI355X fp32: vector (counts packed FMAs) and dense matrix peaks are the same figure


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="gemm8192",
                    choices=["gemm8192", "gemm256", "gemm1024", "gemm_batched", "linear", "linear_prepared", "conv_a_prepared", "linear_bwd", "conv_dw", "conv_dx", "conv_dwx", "conv_dwx_5x5", "gemv", "ragged", "conv_a", "conv_a_5x5", "conv_a_3x3s2", "conv_b",
                             "adam", "softmax_bwd", "matmul_f32",
                             "copy"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary (conv / linear) measurements")
    ap.add_argument("--no-verify", action="store_true")
    ap.add_argument("--no-settle", action="store_true",
                    help="profiling runs: skip the untimed settle phase, so that a kernel trace holds warm-up + timed steps only")
    return ap.parse_args()


def dev(a):
    import numpy as np
    import torch
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


class Workload:
    """name, algorithmic flops and bytes per step, a run() closure, and a verify() closure."""

    def __init__(self, name, flops, bytes_, run, verify, bound, desc, another=None):
        self.name, self.flops, self.bytes, self.run, self.verify, self.bound, self.desc = name, flops, bytes_, run, verify, bound, desc
        # another(): allocates one more independent set of the large operands and the output (same values)
        # and returns a run() closure over it -- for the rotated-buffer timing of the memory-bound workloads
        self.another = another


def tolerance(orc, got, truth, tag):
    import numpy as np
    rms = float(np.sqrt(np.mean(truth ** 2))) or 1.0
    mr, fr = orc.errors(got, truth, rms)
    if not (mr <= 1e-3 and fr <= 1e-4):
        raise SystemExit(f"VERIFY FAILED {tag}: max_rel {mr:.3e} frob_rel {fr:.3e}")
    return {"max_rel": mr, "frob_rel": fr}


def make_workload(name, orc, capi):
    import numpy as np
    import torch
    if name == "gemm8192":
        n = 8192
        A = orc.fill((n, n), 5, "normal", 0.0, 1.0 / np.sqrt(n))
        B = orc.fill((n, n), 1005, "normal", 0.0, 1.0 / np.sqrt(n))
        Ad, Bd = dev(A), dev(B)
        out = torch.empty((n, n), device="cuda")

        run = capi.prepare_gemm(Ad, Bd, out)

        def verify():
            rows = np.sort(np.random.default_rng(5).choice(n, size=16, replace=False))
            truth = np.concatenate([orc.gemm_rows(A, B, int(r), 1, want32=False)[1] for r in rows])
            return tolerance(orc, out[rows.tolist()].cpu().numpy(), truth, name)

        return Workload(name, 2.0 * n ** 3, 3.0 * n * n * 4, run, verify, "mfma",
                        "C[8192,8192] = f16(A)[8192,8192] * f16(B)[8192,8192], fp32 in/out, N(0,1/sqrt(K))"), (A, B)
    if name == "gemm_batched":
        shape = (8, 16, 1024, 1024)
        A = orc.fill(shape, 6, "normal", 0.0, 1.0 / 32.0)
        B = orc.fill(shape, 1006, "normal", 0.0, 1.0 / 32.0)
        Ad, Bd = dev(A), dev(B)
        out = torch.empty(shape, device="cuda")

        def run():
            capi.tensorcore_gemm(Ad, Bd, out=out)

        def verify():
            return tolerance(orc, out[3, 7].cpu().numpy(), orc.gemm_f64(A[3, 7], B[3, 7]), name)

        return Workload(name, 2.0 * 128 * 1024 ** 3, 3.0 * 128 * 1024 * 1024 * 4, run, verify, "mfma",
                        "[8,16,1024,1024] x [8,16,1024,1024] batched over (N,C)"), None
    if name in ("linear", "linear_prepared"):
        Nb, IN, OUT = 4096, 1024, 4096
        X = orc.fill((Nb, IN), 2, "normal", 0.0, 1.0)
        bound = float(np.sqrt(6.0 / IN))
        Wt = orc.fill((OUT, IN), 1002, "uniform", -bound, bound)
        bias = orc.fill((OUT,), 2002, "uniform", -0.03, 0.03)
        Xd, Wd, bd = dev(X), dev(Wt), dev(bias)
        out = torch.empty((Nb, OUT), device="cuda")

        # "_prepared": the fp16 image of W kept in a prepared-operand handle between the calls (a layer whose
        # weights do not change between forward passes)
        handle = capi.Prepared() if name == "linear_prepared" else None
        run = capi.prepare_gemm(Xd, Wd, out, b_trans=True, bias=bd, bias_strides=(0, 1), relu=True, prepared_b=handle)

        def verify():
            truth = np.maximum(orc.gemm_f64(X[:256], Wt, trans_b=True) + bias[None, :].astype(np.float64), 0)
            return tolerance(orc, out[:256].cpu().numpy(), truth, name)

        def another():
            return capi.prepare_gemm(Xd.clone(), Wd.clone(), torch.empty_like(out), b_trans=True, bias=bd, bias_strides=(0, 1), relu=True,
                                     prepared_b=capi.Prepared() if handle is not None else None)

        return Workload(name, 2.0 * Nb * IN * OUT, 4.0 * (Nb * IN + IN * OUT + OUT + Nb * OUT), run, verify, "mfma",
                        "Linear X[4096,1024] W[4096,1024]^T + bias, ReLU" + (", fp16 image of W kept between calls" if handle else ""),
                        another), None
    if name == "linear_bwd":
        # backward of Model::Linear at the L config: W[1,1,OUT,IN] * x[n,1,IN,1] -> dW += dY^T X, dx += dY W
        Nb, IN, OUT = 4096, 1024, 4096
        X = orc.fill((Nb, 1, IN, 1), 2, "normal", 0.0, 1.0)
        bound = float(np.sqrt(6.0 / IN))
        Wt = orc.fill((1, 1, OUT, IN), 1002, "uniform", -bound, bound)
        dY = orc.fill((Nb, 1, OUT, 1), 3002, "normal", 0.0, 1.0)
        Xd, Wd, dYd = dev(X), dev(Wt), dev(dY)
        dW, dX = torch.zeros((1, 1, OUT, IN), device="cuda"), torch.zeros((Nb, 1, IN, 1), device="cuda")

        def run():
            capi.matmul_backward(dW, dX, Wd, Xd, dYd)

        def verify():
            # gradients accumulate over the timed calls: measure one call from zero
            dW.zero_(); dX.zero_()
            run()
            dyr, xr, wr = (orc.round_f16(t).astype(np.float64) for t in (dY, X, Wt))
            t_dW = dyr.reshape(Nb, OUT)[:, :128].T @ xr.reshape(Nb, IN)
            t_dX = dyr.reshape(Nb, OUT)[:128] @ wr.reshape(OUT, IN)
            a = tolerance(orc, dW.reshape(OUT, IN)[:128].cpu().numpy(), t_dW, name + " dW")
            b = tolerance(orc, dX.reshape(Nb, IN)[:128].cpu().numpy(), t_dX, name + " dx")
            return {k: max(a[k], b[k]) for k in a}

        # operands once, gradients read and written ("+=")
        return Workload(name, 2 * 2.0 * Nb * IN * OUT, 4.0 * (Nb * OUT + Nb * IN + OUT * IN + 2 * OUT * IN + 2 * Nb * IN),
                        run, verify, "mfma", "Linear backward: dW[4096,1024] += dY^T X, dx[4096,1024] += dY W (n=4096)"), None
    if name == "conv_dx":
        # data gradient of the CA convolution as one call: dx[16,64,128,128] += conv^T(dy[16,128,128,128], w)
        N, C, H, W, O = 16, 64, 128, 128, 128
        dy = orc.fill((N, O, H, W), 4104, "normal", 0.0, 1.0)
        w = orc.fill((O, C, 3, 3), 1004, "normal", 0.0, float(np.sqrt(2.0 / (C * 9))))
        w_ref = orc.weights_oihw_to_ref(w)
        dyd, wd = dev(dy), dev(w_ref)
        dxd = torch.zeros((N, C, H, W), device="cuda")

        def run():
            capi.conv2d_backward_data(dxd, dyd, wd, 3, 3, 1, 1, accumulate=True)

        def verify():
            dxd.zero_()
            run()
            # fp64 truth for the first image: mirrored convolution of the fp16-rounded operands
            dyr = orc.round_f16(dy[:1]).astype(np.float64)
            wt = orc.round_f16(w_ref).astype(np.float64)[0, 0].reshape(C, 3, 3, O)
            truth = np.zeros((1, C, H, W))
            for r in range(3):
                for sx in range(3):
                    g = np.einsum("nohw,co->nchw", dyr, wt[:, r, sx, :])
                    h0, w0 = r - 1, sx - 1
                    hs, ws = slice(max(0, -h0), min(H, H - h0)), slice(max(0, -w0), min(W, W - w0))
                    truth[:, :, hs.start + h0:hs.stop + h0, ws.start + w0:ws.stop + w0] += g[:, :, hs, ws]
            return tolerance(orc, dxd[:1].cpu().numpy(), truth, name)

        return Workload(name, 2.0 * N * H * W * C * 9 * O, 4.0 * (N * O * H * W + O * C * 9 + 2 * N * C * H * W), run, verify,
                        "hbm", "Conv2d data gradient: dx[16,64,128,128] += dy[16,128,128,128] (*) mirrored w[128,64,3,3]"), None
    if name == "conv_dwx_5x5":
        # weight gradient of a 5x5 convolution of the CA shape straight from x and dy (the gather kernel)
        N, C, H, W, O, K = 16, 64, 128, 128, 128, 5
        x = orc.fill((N, C, H, W), 4, "normal", 0.0, 1.0)
        dy = orc.fill((N, O, H, W), 4104, "normal", 0.0, 1.0)
        xd, dyd = dev(x), dev(dy)
        dwd = torch.zeros((1, 1, C * K * K, O), device="cuda")

        def run():
            capi.conv2d_backward_weights(dwd, xd, dyd, K, K, 1, 2)

        def verify():
            dwd.zero_()
            run()
            xr = np.pad(orc.round_f16(x[:, :2]).astype(np.float64), ((0, 0), (0, 0), (2, 2), (2, 2)))
            dyr = orc.round_f16(dy).astype(np.float64)
            truth = np.zeros((2, K, K, O))
            for r in range(K):
                for sx in range(K):
                    truth[:, r, sx, :] = np.einsum("nchw,nohw->co", xr[:, :, r:r + H, sx:sx + W], dyr)
            return tolerance(orc, dwd.reshape(C, K * K, O)[:2].cpu().numpy().reshape(-1), truth.reshape(-1), name)

        return Workload(name, 2.0 * N * H * W * C * K * K * O, 4.0 * (N * C * H * W + N * O * H * W + 2 * C * K * K * O), run, verify,
                        "hbm", "Conv2d weight gradient, 5x5 s1 p2: dW[1600,128] += x[16,64,128,128] (*) dy[16,128,128,128], no column matrix"), None
    if name == "conv_dwx":
        # weight gradient of the CA convolution straight from x and dy (no column matrix)
        N, C, H, W, O = 16, 64, 128, 128, 128
        x = orc.fill((N, C, H, W), 4, "normal", 0.0, 1.0)
        dy = orc.fill((N, O, H, W), 4104, "normal", 0.0, 1.0)
        xd, dyd = dev(x), dev(dy)
        dwd = torch.zeros((1, 1, C * 9, O), device="cuda")

        def run():
            capi.conv2d_backward_weights(dwd, xd, dyd, 3, 3, 1, 1)

        def verify():
            dwd.zero_()
            run()
            # fp64 truth for the first 4 input channels (all taps, all output channels)
            xr = np.pad(orc.round_f16(x[:, :4]).astype(np.float64), ((0, 0), (0, 0), (1, 1), (1, 1)))
            dyr = orc.round_f16(dy).astype(np.float64)
            truth = np.zeros((4, 3, 3, O))
            for r in range(3):
                for sx in range(3):
                    truth[:, r, sx, :] = np.einsum("nchw,nohw->co", xr[:, :, r:r + H, sx:sx + W], dyr)
            return tolerance(orc, dwd.reshape(C, 9, O)[:4].cpu().numpy().reshape(-1), truth.reshape(-1), name)

        return Workload(name, 2.0 * N * H * W * C * 9 * O, 4.0 * (N * C * H * W + N * O * H * W + 2 * C * 9 * O), run, verify,
                        "hbm", "Conv2d weight gradient: dW[576,128] += x[16,64,128,128] (*) dy[16,128,128,128], no column matrix"), None
    if name == "conv_dw":
        # weight gradient of the CA convolution from its column matrix: dW[576,128] += sum_n col_n^T dZ_n,
        # the batch reduction folded into one contraction of length 16 * 16384
        N, P, CKK, O = 16, 128 * 128, 64 * 9, 128
        col = orc.fill((N, 1, P, CKK), 4004, "normal", 0.0, 1.0)
        dZ = orc.fill((N, 1, P, O), 4005, "normal", 0.0, 1.0)
        Wr = torch.zeros((1, 1, CKK, O), device="cuda")
        cold, dZd = dev(col), dev(dZ)
        dWd = torch.zeros((1, 1, CKK, O), device="cuda")

        def run():
            capi.matmul_backward(None, dWd, cold, Wr, dZd)

        def verify():
            dWd.zero_()
            run()
            # every output needs the whole contraction: fp64 truth for the first 48 rows of dW
            cr = orc.round_f16(col).reshape(N * P, CKK)[:, :48].astype(np.float64)
            zr = orc.round_f16(dZ).reshape(N * P, O).astype(np.float64)
            truth = cr.T @ zr
            return tolerance(orc, dWd.reshape(CKK, O)[:48].cpu().numpy(), truth, name)

        return Workload(name, 2.0 * N * P * CKK * O, 4.0 * (N * P * CKK + N * P * O + 2 * CKK * O), run, verify, "hbm",
                        "Conv weight gradient: dW[576,128] += col[16x16384,576]^T dZ[16x16384,128]"), None
    if name == "gemv":
        a = orc.fill((1, 4096), 4, "uniform", -1.0, 1.0)
        Bm = orc.fill((4096, 4096), 1004, "uniform", -1.0, 1.0)
        ad, Bd = dev(a), dev(Bm)
        out = torch.empty((1, 4096), device="cuda")

        run = capi.prepare_gemm(ad, Bd, out)

        def verify():
            return tolerance(orc, out.cpu().numpy(), orc.gemm_f64(a, Bm), name)

        def another():
            return capi.prepare_gemm(ad.clone(), Bd.clone(), torch.empty_like(out))

        return Workload(name, 2.0 * 4096 * 4096, 4.0 * (4096 + 4096 * 4096 + 4096), run, verify, "hbm",
                        "A[1,4096] * B[4096,4096]", another), None
    if name in ("gemm256", "gemm1024"):
        n = 256 if name == "gemm256" else 1024
        A = orc.fill((n, n), 0, "uniform", -1.0, 1.0)
        B = orc.fill((n, n), 1000, "uniform", -1.0, 1.0)
        Ad, Bd = dev(A), dev(B)
        out = torch.empty((n, n), device="cuda")

        run = capi.prepare_gemm(Ad, Bd, out)

        def verify():
            return tolerance(orc, out.cpu().numpy(), orc.gemm_f64(A, B), name)

        return Workload(name, 2.0 * n ** 3, 4.0 * 3 * n * n, run, verify, "mfma", f"A[{n},{n}] * B[{n},{n}], U[-1,1]"), None
    if name == "ragged":
        A = orc.fill((1000, 777), 3, "uniform", -1.0, 1.0)
        B = orc.fill((777, 513), 1003, "uniform", -1.0, 1.0)
        Ad, Bd = dev(A), dev(B)
        out = torch.empty((1000, 513), device="cuda")

        run = capi.prepare_gemm(Ad, Bd, out)

        def verify():
            return tolerance(orc, out.cpu().numpy(), orc.gemm_f64(A, B), name)

        return Workload(name, 2.0 * 1000 * 777 * 513, 4.0 * (1000 * 777 + 777 * 513 + 1000 * 513), run, verify, "mfma",
                        "A[1000,777] * B[777,513]"), None
    if name in ("conv_a", "conv_b", "conv_a_prepared"):
        prepared = capi.Prepared() if name == "conv_a_prepared" else None
        if name != "conv_b":
            N, C, H, W, O = 16, 64, 128, 128, 128
            x = orc.fill((N, C, H, W), 4, "normal", 0.0, 1.0)
        else:
            N, C, H, W, O = 10, 3, 1024, 1024, 1
            x = orc.fill((N, C, H, W), 14, "uniform", 0.0, 1.0)
        w = orc.fill((O, C, 3, 3), 1004 if name != "conv_b" else 1014, "normal", 0.0, float(np.sqrt(2.0 / (C * 9))))
        bias = orc.fill((O,), 2004 if name != "conv_b" else 2014, "uniform", -0.03, 0.03)
        xd, wd, bd = dev(x), dev(orc.weights_oihw_to_ref(w)), dev(bias)
        out = torch.empty((N, O, H, W), device="cuda")

        def run():
            capi.conv2d_forward(xd, wd, bd, 3, 3, 1, 1, bias_strides=(0, 1), relu=True, out=out, prepared_w=prepared)

        def verify():
            truth = orc.conv2d_direct_f64(x[:1], w, bias, 1, 1, relu=True)
            return tolerance(orc, out[:1].cpu().numpy(), truth, name)

        def another():
            x2, out2 = xd.clone(), torch.empty_like(out)

            def run2():
                capi.conv2d_forward(x2, wd, bd, 3, 3, 1, 1, bias_strides=(0, 1), relu=True, out=out2, prepared_w=prepared)
            return run2

        flops = 2.0 * N * H * W * C * 9 * O
        bytes_ = 4.0 * (N * C * H * W + O * C * 9 + O + N * O * H * W)
        return Workload(name, flops, bytes_, run, verify, "hbm",
                        f"Conv2d x[{N},{C},{H},{W}] w[{O},{C},3,3] s1 p1 + bias + ReLU" +
                        (", fp16 image of the weights kept between calls" if prepared else ""), another), None
    if name in ("conv_a_5x5", "conv_a_3x3s2"):
        # the CA tensor through the kernel that takes any kernel extent and stride (no column matrix)
        N, C, H, W, O = 16, 64, 128, 128, 128
        K, stride, pad = (5, 1, 2) if name == "conv_a_5x5" else (3, 2, 1)
        Ho, Wo = (H + 2 * pad - K) // stride + 1, (W + 2 * pad - K) // stride + 1
        x = orc.fill((N, C, H, W), 4, "normal", 0.0, 1.0)
        w = orc.fill((O, C, K, K), 1005, "normal", 0.0, float(np.sqrt(2.0 / (C * K * K))))
        bias = orc.fill((O,), 2005, "uniform", -0.03, 0.03)
        xd, wd, bd = dev(x), dev(orc.weights_oihw_to_ref(w)), dev(bias)
        out = torch.empty((N, O, Ho, Wo), device="cuda")

        def run():
            capi.conv2d_forward(xd, wd, bd, K, K, stride, pad, bias_strides=(0, 1), relu=True, out=out)

        def verify():
            truth = orc.conv2d_direct_f64(x[:1], w, bias, stride, pad, relu=True)
            return tolerance(orc, out[:1].cpu().numpy(), truth, name)

        flops = 2.0 * N * Ho * Wo * C * K * K * O
        bytes_ = 4.0 * (N * C * H * W + O * C * K * K + O + N * O * Ho * Wo)
        return Workload(name, flops, bytes_, run, verify, "hbm",
                        f"Conv2d x[{N},{C},{H},{W}] w[{O},{C},{K},{K}] s{stride} p{pad} + bias + ReLU"), None
    if name == "adam":
        # opt::Adam::step over 2^26 parameters: data, m, v read and written, the gradient read
        n = 1 << 26
        gen = torch.Generator(device="cuda").manual_seed(5)
        d = torch.randn(n, device="cuda", generator=gen)
        g = torch.randn(n, device="cuda", generator=gen)
        m = torch.zeros(n, device="cuda")
        v = torch.zeros(n, device="cuda")
        step = [0]

        def run():
            step[0] += 1
            capi.adam_step(d, m, v, g, 1e-3, 0.9, 0.999, 1e-8, step[0])

        def verify():
            # one more step on a slice of the live state against the CPU restatement
            k = 1 << 16
            hs = [t[:k].cpu().numpy().copy() for t in (d, m, v, g)]
            ds, ms_, vs = d[:k].clone(), m[:k].clone(), v[:k].clone()
            capi.adam_step(ds, ms_, vs, g[:k], 1e-3, 0.9, 0.999, 1e-8, step[0] + 1)
            do, mo, vo = orc.adam_step(hs[0], hs[1], hs[2], hs[3], 1e-3, 0.9, 0.999, 1e-8, step[0] + 1)
            ok = (np.allclose(ds.cpu().numpy(), do, rtol=1e-5, atol=1e-6) and np.allclose(ms_.cpu().numpy(), mo, rtol=1e-6, atol=1e-7)
                  and np.allclose(vs.cpu().numpy(), vo, rtol=1e-6, atol=1e-7))
            if not ok:
                raise SystemExit("VERIFY FAILED adam")
            return {"allclose_1e-5": True}

        return Workload(name, 12.0 * n, 28.0 * n, run, verify, "hbm", "Adam step over 2^26 fp32 parameters"), None
    if name == "softmax_bwd":
        # SoftmaxNode::backward for 64 vectors of 4096 classes: Jacobian x gradient, fp16-rounded operands,
        # the Jacobian never in memory (the two-call spelling would write and read 64 x 64 MiB)
        n, batch = 4096, 64
        x = orc.fill((batch, 1, n, 1), 6, "uniform", -4.0, 4.0)
        so = orc.softmax(x)
        dy = orc.fill((batch, 1, n, 1), 1006, "uniform", -1.0, 1.0)
        sd, dyd = dev(so), dev(dy)
        out = [None]

        def run():
            out[0] = capi.softmax_backward(sd, dyd)

        def verify():
            want = orc.softmax_backward(so[:2], dy[:2])
            if not np.array_equal(out[0][:2].cpu().numpy(), want):
                raise SystemExit("VERIFY FAILED softmax_bwd")
            return {"bit_exact": True}

        return Workload(name, 2.0 * n * n * batch, 12.0 * n * batch, run, verify, "valu_fp32",
                        "softmax backward, 64 vectors x 4096 (fp32 VALU kernel, fp16-rounded operands)"), None
    if name == "matmul_f32":
        # Tensor::operator*: fp32-exact product, one FMA chain per output in ascending k (VALU kernel)
        M = 2048
        A = orc.fill((M, M), 7, "uniform", -1.0, 1.0)
        B = orc.fill((M, M), 1007, "uniform", -1.0, 1.0)
        Ad, Bd = dev(A).reshape(1, 1, M, M), dev(B).reshape(1, 1, M, M)
        out = torch.empty((1, 1, M, M), device="cuda")

        def run():
            capi.matmul_f32(Ad, Bd, out=out)

        def verify():
            rows = 16
            want = orc.general_matmul(A[:rows].reshape(1, 1, rows, M), B.reshape(1, 1, M, M))
            if not np.array_equal(out[0, 0, :rows].cpu().numpy(), want.reshape(rows, M)):
                raise SystemExit("VERIFY FAILED matmul_f32")
            return {"bit_exact": True}

        return Workload(name, 2.0 * M ** 3, 12.0 * M * M, run, verify, "mfma_fp32",
                        "fp32-exact A[2048,2048] * B[2048,2048] (fp32 MFMA kernel; fp32 matrix peak 157.3 TFLOP/s)"), None
    if name == "copy":
        # Calibration only: a plain device copy of known size (1 GiB read + 1 GiB written), so that
        # rocprofv3's FETCH_SIZE / WRITE_SIZE readings can be scaled to bytes.
        n = 1 << 28
        src = torch.rand(n, device="cuda")
        dst = torch.empty(n, device="cuda")

        def run():
            dst.copy_(src)

        def verify():
            assert torch.equal(dst, src)
            return {"max_rel": 0.0, "frob_rel": 0.0}

        return Workload(name, 0.0, 8.0 * n, run, verify, "hbm", "torch elementwise copy of 2^28 fp32 (calibration)"), None
    raise ValueError(name)


SETTLE_SECONDS = 0.25


def settle(run, seconds=SETTLE_SECONDS):
    """Untimed: keeps the GPU on the workload for a quarter of a second before the warm-up steps. After an
    idle period the power management first overshoots and then throttles (the 8192^3 kernel runs 0.93, 1.18,
    ... ms over its first twenty calls before it levels out at 0.90 ms); the metric is the steady rate."""
    import torch
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            run()
        torch.cuda.synchronize()


def time_steps(wl, steps, warmup, do_settle=True):
    """Times exactly `steps` runs with HIP events recorded on the stream the kernels are
    launched on (torch's current stream), bracketed by device synchronisation."""
    import torch
    if do_settle:
        settle(wl.run)
    for _ in range(warmup):
        wl.run()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        wl.run()
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return start.elapsed_time(stop) / steps, wall * 1e3 / steps      # ms per step (device events, host wall)


def per_step_stats(wl, steps):
    """A second loop of `steps` runs with an event between every two of them: median, min and max of the
    single steps in ms. The event packets sit between the kernels of neighbouring steps, so for steps of a
    few microseconds these figures carry that gap; the mean of time_steps() (one event pair around the whole
    loop) does not and stays the reported `ms_per_step`."""
    import torch
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    ev[0].record()
    for i in range(steps):
        wl.run()
        ev[i + 1].record()
    torch.cuda.synchronize()
    ts = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(steps))
    return {"median_ms": ts[len(ts) // 2], "min_ms": ts[0], "max_ms": ts[-1], "steps": steps}


class PowerClockSampler:
    """Best effort: reads the GPU's package power and shader clock from sysfs in a background thread while a
    loop runs (amdgpu's hwmon power1_input / power1_average, pp_dpm_sclk). Figures are None where the files are
    not there or not readable."""

    def __init__(self):
        import glob
        dev = "/sys/class/drm/card*/device/"
        self.pw = (glob.glob(dev + "hwmon/hwmon*/power1_input") + glob.glob(dev + "hwmon/hwmon*/power1_average"))[:1]
        self.cap = glob.glob(dev + "hwmon/hwmon*/power1_cap")[:1]
        self.ck = glob.glob(dev + "pp_dpm_sclk")[:1]
        self.power, self.clock, self._stop, self._th = [], [], False, None

    def _loop(self):
        while not self._stop:
            try:
                if self.pw:
                    self.power.append(int(open(self.pw[0]).read()) / 1e6)
                if self.ck:
                    cur = [l for l in open(self.ck[0]).read().splitlines() if "*" in l]
                    if cur:
                        self.clock.append(float(cur[0].split(":")[1].lower().replace("mhz", "").replace("*", "").strip()))
            except (OSError, ValueError, IndexError):
                pass
            time.sleep(0.01)

    def __enter__(self):
        import threading
        self.power, self.clock, self._stop = [], [], False
        self._th = threading.Thread(target=self._loop, daemon=True)
        self._th.start()
        return self

    def __exit__(self, *a):
        self._stop = True
        self._th.join()

    @staticmethod
    def _median(v):
        v = sorted(v)
        return v[len(v) // 2] if v else None

    def result(self, skip=0.25):
        """medians over the samples after the first quarter (the ramp after an idle period)"""
        p, c = self.power[int(len(self.power) * skip):], self.clock[int(len(self.clock) * skip):]
        cap = None
        try:
            cap = int(open(self.cap[0]).read()) / 1e6 if self.cap else None
        except (OSError, ValueError):
            pass
        return {"power_W": self._median(p), "sclk_MHz": self._median(c), "power_cap_W": cap, "samples": len(p)}


def box_ceilings(capi, wl_run):
    """What this box sustains: (i) a register-only MFMA loop (random fp16 operands; zeros for comparison) with the
    clock the chip held under it, (ii) a plain 16-byte copy over rotated buffers (nothing served by the caches)
    and over the same buffers, (iii) package power and shader clock while the headline workload runs back to
    back for about a second."""
    import ctypes as C
    import torch
    lib = capi.load()
    out = {}
    ws = torch.zeros(65536 // 4, dtype=torch.float32, device="cuda")
    stream = C.c_void_p(int(torch.cuda.current_stream().cuda_stream))
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    passes = 4000
    for zero, key in ((0, "mfma_loop_random_operands"), (1, "mfma_loop_zero_operands")):
        for _ in range(4):                                            # settle: ~40 ms of the loop
            capi.check(lib.nzhip_probe_mfma(passes, zero, ws.data_ptr(), 65536, stream))
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = 10
        e0.record()
        for _ in range(reps):
            capi.check(lib.nzhip_probe_mfma(passes, zero, ws.data_ptr(), 65536, stream))
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        st = ws[: 2 * cus * 2].view(torch.int64).cpu().tolist()       # (shader ticks, 100 MHz ticks) per workgroup
        ratios = sorted(st[2 * i] / st[2 * i + 1] for i in range(cus) if st[2 * i + 1] > 0)
        out[key] = {"TFLOP/s": cus * 4 * passes * 64 * 16384.0 / ms / 1e9,
                    "clock_MHz": 100.0 * ratios[len(ratios) // 2] if ratios else None,
                    "desc": f"{cus} workgroups x 4 waves x {passes} x 64 v_mfma_f32_16x16x32_f16 from registers"}
    # copy: 4 source/destination pairs of 256 MiB each (2 GiB in all) used round robin, and one pair reused
    n = 1 << 26
    pairs = [(torch.rand(n, device="cuda"), torch.empty(n, device="cuda")) for _ in range(4)]

    def copy_loop(k, reps):
        for i in range(8):
            capi.check(lib.nzhip_probe_copy(pairs[i % k][1].data_ptr(), pairs[i % k][0].data_ptr(), 4 * n, stream))
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(reps):
            capi.check(lib.nzhip_probe_copy(pairs[i % k][1].data_ptr(), pairs[i % k][0].data_ptr(), 4 * n, stream))
        e1.record()
        torch.cuda.synchronize()
        return 8.0 * n * reps / (e0.elapsed_time(e1) * 1e-3) / 1e9

    out["copy_rotated_GB/s"] = copy_loop(4, 40)
    assert torch.equal(pairs[3][1], pairs[3][0])
    del pairs[1:]
    out["copy_same_buffers_256MiB_GB/s"] = copy_loop(1, 40)
    n_small = 1 << 24                                                  # 64 MiB + 64 MiB: fits the memory-side cache
    src, dst = pairs[0][0][:n_small], pairs[0][1][:n_small]
    for _ in range(8):
        capi.check(lib.nzhip_probe_copy(dst.data_ptr(), src.data_ptr(), 4 * n_small, stream))
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(100):
        capi.check(lib.nzhip_probe_copy(dst.data_ptr(), src.data_ptr(), 4 * n_small, stream))
    e1.record()
    torch.cuda.synchronize()
    out["copy_same_buffers_64MiB_GB/s"] = 8.0 * n_small * 100 / (e0.elapsed_time(e1) * 1e-3) / 1e9
    del pairs, src, dst
    torch.cuda.empty_cache()
    with PowerClockSampler() as smp:
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 1.0:
            for _ in range(16):
                wl_run()
            torch.cuda.synchronize()
    out["under_headline_workload"] = smp.result()
    return out


ROTATE_MIN_BYTES = 640 << 20


def time_rotated(wl, steps, warmup):
    """Steady-state loop over k >= 4 independent operand/output sets, more than 640 MiB in total, used round
    robin: by the time a set comes round again every byte of it has left the 32 MiB of L2 and the 256 MiB
    memory-side cache, so the rate is that of HBM. Returns (ms per step, k)."""
    import torch
    k = max(4, int(ROTATE_MIN_BYTES // wl.bytes) + 1)
    runs = [wl.run] + [wl.another() for _ in range(k - 1)]
    steps = max(steps, 2 * k)
    for i in range(max(warmup, k)):
        runs[i % k]()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        runs[i % k]()
    stop.record()
    torch.cuda.synchronize()
    del runs
    return start.elapsed_time(stop) / steps, k


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    import platform
    return platform.processor() or "unknown"


def time_cold(wl, iters=10):
    """One run at a time with the caches emptied in between: a 1 GiB device copy (512 MiB read,
    512 MiB written) runs before each timed run, so neither the 32 MiB of L2 nor the 256 MiB
    memory-side cache still holds the workload's operands from the run before. Returns the median
    of `iters` single-run event timings in ms."""
    import torch
    n = 1 << 27
    src, dst = torch.empty(n, device="cuda"), torch.empty(n, device="cuda")
    src.fill_(1.0)
    ts = []
    for _ in range(iters):
        dst.copy_(src)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        wl.run()
        stop.record()
        torch.cuda.synchronize()
        ts.append(start.elapsed_time(stop))
    ts.sort()
    del src, dst
    return ts[len(ts) // 2]


def cpu_baseline_gemm(orc, A, B, rows=8192):
    """The oracle (a port of the reference semantics, OpenMP over the host cores the process may
    use) on the same workload: all `rows` rows of the 8192^3 product, best of 3."""
    n = A.shape[1]
    orc.gemm_rows(A, B, 0, 64, want64=False)                      # warm-up (thread pool, page faults)
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        orc.gemm_rows(A, B, 0, rows, want64=False)
        dt = time.perf_counter() - t0
        best = dt if best is None or dt < best else best
    return {"value": 2.0 * rows * n * B.shape[1] / best / 1e12, "unit": "TFLOP/s", "cores": orc.num_threads(),
            "cpu_model": cpu_model(), "kind": "port", "sample": f"the whole 8192^3 GEMM ({rows}x8192x8192 incl. rounding both operands), best of 3, {best:.2f} s each"}


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU only (the path shards by rows or batch members with no "
              "exchange between GPUs); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    from neuzephyr_amd import capi
    from oracle import oracle as orc     # checker + cpu_baseline only
    capi.load()

    wl, host_ops = make_workload(args.workload, orc, capi)
    ms_dev, ms_wall = time_steps(wl, args.steps, args.warmup, not args.no_settle)
    step_stats = per_step_stats(wl, args.steps)
    verified = None if args.no_verify else wl.verify()

    tflops = wl.flops / (ms_dev * 1e-3) / 1e12
    gbps = wl.bytes / (ms_dev * 1e-3) / 1e9
    # HBM bytes per step as read from rocprofv3 FETCH_SIZE / WRITE_SIZE (scaled by a copy kernel of
    # known size); the figures are kept, with the commands that produced them, under profiles/.
    traffic = None
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            traffic = json.load(f).get(args.workload, {}).get("bytes_per_step")
    except OSError:
        pass
    scope = ("whole step = every kernel the call launches (for gemm8192: the kernel that rounds the first stage of "
             "the operands + the MFMA kernel, which rounds the rest inside its k loops); per-kernel durations are "
             "in profiles/")
    if wl.bound == "mfma":
        roofline = {"bound": "mfma", "achieved": tflops, "peak": PEAK_TFLOPS_FP16, "unit": "TFLOP/s",
                    "frac": tflops / PEAK_TFLOPS_FP16, "traffic": traffic, "scope": scope}
    elif wl.bound in ("valu_fp32", "mfma_fp32"):        # the fp32 kernels (not the default workload)
        roofline = {"bound": wl.bound, "achieved": tflops, "peak": PEAK_TFLOPS_FP32, "unit": "TFLOP/s",
                    "frac": tflops / PEAK_TFLOPS_FP32, "traffic": traffic, "scope": scope}
    else:
        roofline = {"bound": "hbm", "achieved": gbps, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                    "frac": gbps / PEAK_HBM_GBPS, "traffic": traffic, "scope": scope}

    extra = {}
    if args.workload == "gemm8192" and not args.no_extra:
        for name in ("conv_b", "conv_a", "conv_a_prepared", "conv_a_5x5", "conv_a_3x3s2", "linear", "linear_prepared", "gemv", "ragged", "gemm256", "gemm1024", "gemm_batched", "linear_bwd", "conv_dw", "conv_dx", "conv_dwx", "conv_dwx_5x5", "adam",
                     "softmax_bwd", "matmul_f32"):
            torch.cuda.empty_cache()
            w2, _ = make_workload(name, orc, capi)
            ms2, _ = time_steps(w2, max(10, args.steps // 2), max(3, args.warmup // 2))
            st2 = per_step_stats(w2, max(10, args.steps // 2))
            v2 = None if args.no_verify else w2.verify()
            ms_cold = time_cold(w2)
            extra[name] = {"ms": ms2, "per_step_events": st2, "ms_cold_caches": ms_cold, "GB/s_cold_caches": w2.bytes / ms_cold / 1e6,
                           "TFLOP/s": w2.flops / ms2 / 1e9, "GB/s": w2.bytes / ms2 / 1e6,
                           "frac_mfma_peak": w2.flops / ms2 / 1e9 / PEAK_TFLOPS_FP16,
                           "frac_hbm_peak": w2.bytes / ms2 / 1e6 / PEAK_HBM_GBPS, "verified": v2, "workload": w2.desc}
            if w2.another is not None:
                # the HBM figure proper: operands rotated through more memory than the caches hold; the
                # same-buffer loop above re-reads a working set that the 256 MiB memory-side cache can serve
                ms_rot, k = time_rotated(w2, max(10, args.steps // 2), max(3, args.warmup // 2))
                e = extra[name]
                e["frac_hbm_peak_same_buffers"] = e["frac_hbm_peak"]
                e.update({"ms_rotated_buffers": ms_rot, "rotated_sets": k, "rotated_bytes": k * w2.bytes,
                          "GB/s_rotated_buffers": w2.bytes / ms_rot / 1e6,
                          "frac_hbm_peak": w2.bytes / ms_rot / 1e6 / PEAK_HBM_GBPS,
                          "frac_mfma_peak_rotated_buffers": w2.flops / ms_rot / 1e9 / PEAK_TFLOPS_FP16})
                torch.cuda.empty_cache()
            if w2.bound in ("valu_fp32", "mfma_fp32"):
                del extra[name]["frac_mfma_peak"]
                key = "frac_fp32_vector_peak" if w2.bound == "valu_fp32" else "frac_fp32_matrix_peak"
                extra[name][key] = w2.flops / ms2 / 1e9 / PEAK_TFLOPS_FP32
            del w2

    if args.workload == "gemm8192" and not args.no_extra:
        # the reference's README network (batch 10 x 3 x 1024 x 1024) through the C++ nz:: layer, one Adam
        # training step; a child process of its own (host wall clock around a device synchronisation)
        exe = os.path.join(ROOT, "neuzephyr_amd", "nz", "examples", "readme_example")
        if os.path.exists(exe):
            torch.cuda.empty_cache()
            import subprocess
            try:
                out = subprocess.run([exe, "10", "3"], capture_output=True, text=True, timeout=120)
                extra["readme_example_training_step"] = (json.loads(out.stdout.strip().splitlines()[-1]) if out.returncode == 0
                                                         else {"error": out.stderr[-300:]})
            except (subprocess.TimeoutExpired, ValueError, IndexError) as e:
                extra["readme_example_training_step"] = {"error": str(e)[:300]}

    if args.workload == "gemm8192" and not args.no_extra:
        # single layers through the C++ nz:: API (Model::forward()), with and without the kept weight images
        exe = os.path.join(ROOT, "neuzephyr_amd", "nz", "examples", "layer_bench")
        if os.path.exists(exe):
            torch.cuda.empty_cache()
            import subprocess
            try:
                out = subprocess.run([exe, "200", "20"], capture_output=True, text=True, timeout=120)
                extra["layers_through_model"] = (json.loads(out.stdout.strip().splitlines()[-1]) if out.returncode == 0
                                                         else {"error": out.stderr[-300:]})
            except (subprocess.TimeoutExpired, ValueError, IndexError) as e:
                extra["layers_through_model"] = {"error": str(e)[:300]}

    ceilings = None
    if args.workload == "gemm8192" and not args.no_extra:
        torch.cuda.empty_cache()
        ceilings = box_ceilings(capi, wl.run)
        mf, cp = ceilings["mfma_loop_random_operands"]["TFLOP/s"], ceilings["copy_rotated_GB/s"]
        roofline["frac_of_box_mfma_loop"] = tflops / mf
        for e in extra.values():
            if isinstance(e, dict) and "TFLOP/s" in e and "frac_mfma_peak" in e:
                e["frac_of_box_mfma_loop"] = e["TFLOP/s"] / mf
            if isinstance(e, dict) and "GB/s_rotated_buffers" in e:
                e["frac_of_box_copy_rotated"] = e["GB/s_rotated_buffers"] / cp

    cpu = None
    if args.workload == "gemm8192" and not args.no_cpu_baseline:
        cpu = cpu_baseline_gemm(orc, *host_ops)

    line = {
        "metric": "fp16-MFMA TFLOP/s (% peak) on 8192^3 GEMM; Conv2d fwd GB/s (% HBM peak)",
        "value": gbps if wl.bound == "hbm" else tflops,
        "unit": "GB/s" if wl.bound == "hbm" else "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_dev, "ms_per_step_host_wall": ms_wall, "per_step_events": step_stats,
        "untimed_settle_s_before_warmup": 0.0 if args.no_settle else SETTLE_SECONDS,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "dtype_note": "fp32 operands rounded to fp16 (RNE), fp16 MFMA, fp32 accumulate and output",
        "data": "synthetic",
        "config": {"workload": args.workload, "desc": wl.desc, "algorithmic_flops": wl.flops,
                   "algorithmic_bytes": wl.bytes},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "box_ceilings": ceilings,
        "verified": verified,
        "conv_and_other_configs": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
