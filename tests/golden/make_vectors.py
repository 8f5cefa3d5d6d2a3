"""Writes tests/golden/w8a8_vectors.npz: inputs and expected outputs of the W8A8 block-FP8 linear path on small
shapes, computed with torch CPU library ops only (casts to bfloat16 / float8_e4m3fn, abs/amax/clamp/div, float64
matmul of dequantised operands) - no code of the oracle or of the HIP library takes part.  The reference ships no
golden vectors for this path (its tests synthesise data and compare against torch-native formulas,
python/sglang/test/test_block_fp8.py:23-48,273-325); these follow the same formulas.

    python tests/golden/make_vectors.py

Cases: activations with outliers, an all-zero group (scale = eps / 448), a group whose amax is exactly 448, values
that fall on e4m3 rounding ties, ragged N (not a multiple of 128).
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def group_quant(x_bf16, group=128, eps=1e-10):
    g = x_bf16.reshape(-1, group)
    amax = g.abs().max(dim=-1, keepdim=True)[0].clamp(min=eps).to(torch.float32)
    s = amax / 448.0
    q = (g / s).clamp(min=-448.0, max=448.0).to(torch.float8_e4m3fn)
    return q.reshape(x_bf16.shape), s.reshape(x_bf16.shape[0], -1)


def block_quant_weight(w_bf16, bn=128, bk=128):
    N, K = w_bf16.shape
    q = torch.empty((N, K), dtype=torch.float8_e4m3fn)
    s = torch.empty(((N + bn - 1) // bn, (K + bk - 1) // bk), dtype=torch.float32)
    for j in range(s.shape[0]):
        for i in range(s.shape[1]):
            t = w_bf16[j * bn:(j + 1) * bn, i * bk:(i + 1) * bk].float()
            sc = t.abs().max().clamp(min=1e-10) / 448.0
            s[j, i] = sc
            q[j * bn:(j + 1) * bn, i * bk:(i + 1) * bk] = (t / sc).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q, s


def dequant_matmul(q, s, wq, ws, bn=128, bk=128):
    a = q.double() * s.double().repeat_interleave(bk, dim=1)[:, :q.shape[1]]
    b = wq.double() * ws.double().repeat_interleave(bn, dim=0)[:wq.shape[0]].repeat_interleave(bk, dim=1)[:, :wq.shape[1]]
    return a @ b.t()


def main():
    gen = torch.Generator().manual_seed(20240607)
    out = {}
    for name, (M, N, K) in {"a": (7, 256, 384), "b": (33, 200, 256), "c": (70, 128, 128)}.items():
        x = torch.randn((M, K), generator=gen) * 3.0
        x[torch.rand((M, K), generator=gen) < 0.002] *= 60.0          # outliers
        x[0, :128] = 0.0                                              # an all-zero group
        x[M - 1, K - 128:] = torch.linspace(-448.0, 448.0, 128)       # amax exactly 448: scale 1
        x[1, :128] = torch.arange(128, dtype=torch.float32) * 1.75     # e4m3 ties after the divide (amax 222.25)
        x = x.bfloat16()
        w = (torch.randn((N, K), generator=gen) * 0.05).bfloat16()
        q, s = group_quant(x)
        wq, ws = block_quant_weight(w)
        y = dequant_matmul(q, s, wq, ws)
        out[name + "_x_bf16_bits"] = x.view(torch.int16).numpy().view(np.uint16)
        out[name + "_q"] = q.view(torch.uint8).numpy()
        out[name + "_s"] = s.numpy()
        if name == "a":
            out[name + "_w_bf16_bits"] = w.view(torch.int16).numpy().view(np.uint16)
        out[name + "_wq"] = wq.view(torch.uint8).numpy()
        out[name + "_ws"] = ws.numpy()
        out[name + "_y"] = y.float().numpy()  # float64 product rounded once to float32
    np.savez_compressed(os.path.join(HERE, "w8a8_vectors.npz"), **out)
    print("wrote", os.path.join(HERE, "w8a8_vectors.npz"), {k: v.shape for k, v in out.items() if k.startswith("c_")})


if __name__ == "__main__":
    main()
