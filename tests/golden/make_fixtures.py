"""Writes the committed golden vectors from this repository's own CPU oracle (never from the reference).
Run from the repository root: python tests/golden/make_fixtures.py"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as O  # noqa: E402
from applied_ai_amd import configs  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def cfg1():
    c = configs.cfg1()
    x, w, logits = c["x"].numpy(), c["w"].numpy(), c["logits"].numpy()
    ids = O.topk(logits, 2)
    perm, m_sizes = O.route(ids, 8)
    x_sorted = x[perm // 2]
    y = O.grouped_gemm(x_sorted, w, m_sizes)
    xb = torch.from_numpy(x_sorted).to(torch.bfloat16).float().numpy()
    wb = torch.from_numpy(w).to(torch.bfloat16).float().numpy()
    yb = O.grouped_gemm(xb, wb, m_sizes)
    # bf16 inputs are stored as their 16-bit patterns (upper half of the fp32 word)
    bits = lambda a: (a.view(np.uint32) >> 16).astype(np.uint16)
    np.savez_compressed(os.path.join(HERE, "cfg1.npz"), logits=logits, ids=ids, perm=perm, m_sizes=m_sizes,
                        offsets=O.offsets(m_sizes), x_sorted_bf16_bits=bits(xb), w_bf16_bits=bits(wb),
                        y_bf16_inputs=yb, y_fp32_inputs_first64rows=y[:64])


def w4a16_tiny():
    """K=256, N=64, M in {1, 16}, both zero-point conventions (splitk_dequant_gemm.py:73-74 uses z + 1)."""
    rng = np.random.default_rng(20240601)
    K, N, g = 256, 64, 128
    q = rng.integers(0, 16, size=(K, N))
    z = rng.integers(0, 16, size=(K // g, N))
    scales = torch.from_numpy(rng.uniform(0.005, 0.02, size=(K // g, N)).astype(np.float32)).to(torch.bfloat16).float().numpy()
    a = torch.from_numpy(rng.standard_normal((16, K)).astype(np.float32)).to(torch.bfloat16).float().numpy()
    qw, qz = O.pack_int4_along_k(q), O.pack_int4_along_n(z)
    out = dict(a=a, qweight=qw, scales=scales, qzeros=qz)
    for zo in (0, 1):
        out[f"c_zo{zo}_m16"] = O.w4a16_gemm(a, qw, scales, qz, g, zo)
        out[f"c_zo{zo}_m1"] = O.w4a16_gemm(a[:1], qw, scales, qz, g, zo)
    np.savez_compressed(os.path.join(HERE, "w4a16_tiny.npz"), **out)


def fp8_block_tiny():
    """G=4, K=256, N=256, 1x128 activation scales and 128x128 weight scales."""
    rng = np.random.default_rng(20240602)
    G, N, K = 4, 256, 256
    m_sizes = np.array([5, 0, 40, 19], dtype=np.int32)
    x = rng.standard_normal((int(m_sizes.sum()), K)).astype(np.float32)
    w = (rng.standard_normal((G * N, K)) * 0.02).astype(np.float32)
    xq, xs = O.fp8_groupwise_quant(x)
    wq, ws = O.fp8_block_quant_weight(w)
    y = O.grouped_gemm_fp8(xq, wq, xs, ws, m_sizes, 1)
    xr, xrs = O.fp8_groupwise_quant(x, 128)
    rs_x = np.abs(x).max(axis=1) / 448.0
    rs_w = np.abs(w).max(axis=1) / 448.0
    xq_r = O.f32_to_e4m3(np.clip(x / rs_x[:, None], -448, 448))
    wq_r = O.f32_to_e4m3(np.clip(w / rs_w[:, None], -448, 448))
    y_row = O.grouped_gemm_fp8(xq_r, wq_r, rs_x, rs_w, m_sizes, 0)
    np.savez_compressed(os.path.join(HERE, "fp8_tiny.npz"), m_sizes=m_sizes, x=x, xq=xq, xs=xs, wq=wq, ws=ws, y_block=y,
                        xq_row=xq_r, wq_row=wq_r, xs_row=rs_x.astype(np.float32), ws_row=rs_w.astype(np.float32), y_row=y_row)


if __name__ == "__main__":
    cfg1()
    w4a16_tiny()
    fp8_block_tiny()
    print("wrote", os.listdir(HERE))
