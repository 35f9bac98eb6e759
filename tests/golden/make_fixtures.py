"""Writes tests/golden/smlm_small.npz: inputs and expected outputs of the SMLM
path for one small case, computed with numpy float64 matmuls and numpy / torch
casts only -- independent of oracle/smlm_oracle.c and of the HIP kernels.

The reference holds no golden vector for this path (its tests/ are end-to-end
throughput scripts without assertions), so these vectors are this build's own.
Case: T=13, h_in=64, h_out=96, r=8, 3 adapters, segment=[0,5,5,9,13] (one
empty segment), adapters [2,0,2,1]; fp32 / fp16 / bf16; forward, and backward
on the first two non-empty partitions.

Run:  python tests/golden/make_fixtures.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
T, H_IN, H_OUT, R, NA = 13, 64, 96, 8, 3
SEG = np.array([0, 5, 5, 9, 13], np.int32)
IDS = np.array([2, 0, 2, 1], np.int32)
TP = np.array([0, 5, 9], np.int32)       # train partitions (rows 0..9)
TP_AD = np.array([2, 2], np.int32)       # both train adapter 2 -> summed gradients


def cast(a, dtype):
    t = torch.from_numpy(np.asarray(a, np.float64))
    if dtype == "fp16":
        return t.to(torch.float16).to(torch.float64).numpy()
    if dtype == "bf16":
        return t.to(torch.float32).to(torch.bfloat16).to(torch.float64).numpy()
    return t.to(torch.float32).to(torch.float64).numpy()


def main():
    rng = np.random.default_rng(20240531)
    out = {"seg": SEG, "ids": IDS, "tp": TP, "tp_ad": TP_AD}
    for dt in ("fp32", "fp16", "bf16"):
        x = cast(rng.standard_normal((T, H_IN)), dt)
        A = [cast(rng.standard_normal((R, H_IN)) / 8.0, dt) for _ in range(NA)]
        B = [cast(rng.standard_normal((H_OUT, R)) / np.sqrt(R), dt) for _ in range(NA)]
        g = cast(rng.standard_normal((T, H_OUT)), dt)
        v = np.zeros((T, R))
        y = np.zeros((T, H_OUT))
        for i in range(len(IDS)):
            a, b = SEG[i], SEG[i + 1]
            v[a:b] = cast(x[a:b] @ A[IDS[i]].T, dt)
            y[a:b] = cast(v[a:b] @ B[IDS[i]].T, dt)
        # backward, layout of the forward: dV = g B, dX = dV A, dA = dV^T x, dB = g^T v
        dx = np.zeros((T, H_IN))
        da = [np.zeros((R, H_IN)) for _ in range(NA)]
        db = [np.zeros((H_OUT, R)) for _ in range(NA)]
        for p in range(len(TP_AD)):
            a, b, ad = TP[p], TP[p + 1], TP_AD[p]
            dv = cast(g[a:b] @ B[ad], dt)
            vv = cast(x[a:b] @ A[ad].T, dt)
            dx[a:b] = cast(dv @ A[ad], dt)
            da[ad] += dv.T @ x[a:b]
            db[ad] += g[a:b].T @ vv
        out[f"{dt}_x"] = x.astype(np.float32)
        out[f"{dt}_A"] = np.stack(A).astype(np.float32)
        out[f"{dt}_B"] = np.stack(B).astype(np.float32)
        out[f"{dt}_g"] = g.astype(np.float32)
        out[f"{dt}_v"] = v.astype(np.float32)
        out[f"{dt}_y"] = y.astype(np.float32)
        out[f"{dt}_dx"] = dx.astype(np.float32)
        out[f"{dt}_dA"] = np.stack([cast(d, dt) for d in da]).astype(np.float32)
        out[f"{dt}_dB"] = np.stack([cast(d, dt) for d in db]).astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "smlm_small.npz"), **out)
    print("wrote", os.path.join(HERE, "smlm_small.npz"))


if __name__ == "__main__":
    main()
