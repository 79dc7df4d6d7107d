#!/usr/bin/env python3
"""Writes tests/golden/vectors.npz: small known-answer cases for the hot-path operators.

The reference holds no expected outputs for this path (its own test prints a checksum,
tests/endpoint.py:85), so these vectors are computed here from the published definitions of the
operators with independent library routines in float64 (numpy matmul / einsum, torch.nn.functional
on CPU) -- not with this repository's oracle and not with its kernels.  tests/test_golden.py
checks both the C oracle (CPU) and the HIP kernels (GPU) against them.

Run from the repository root:  python tests/golden/make_vectors.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F


def main():
    rng = np.random.default_rng(20240607)
    f32 = lambda *s: rng.standard_normal(s).astype(np.float32)
    out = {}

    # GEMM  C = X . W^T + bias, with GELU (cublasSgemm + bias/activation epilogue)
    X, W, b = f32(37, 72), f32(50, 72), f32(50)
    z = X.astype(np.float64) @ W.astype(np.float64).T + b
    out.update(gemm_x=X, gemm_w=W, gemm_b=b, gemm_y=z.astype(np.float32),
               gemm_gelu=F.gelu(torch.from_numpy(z)).numpy().astype(np.float32))

    # convolution 3x3 stride 2 pad 1 + inference batch-norm + ReLU, NHWC in / out
    x, w = f32(2, 9, 8, 16), (f32(24, 16, 3, 3) * 0.1).astype(np.float32)
    g, be, mu = f32(24), f32(24), f32(24)
    var = rng.uniform(0.5, 2.0, 24).astype(np.float32)
    t = F.conv2d(torch.from_numpy(x).double().permute(0, 3, 1, 2), torch.from_numpy(w).double(), stride=2, padding=1)
    tb = F.batch_norm(t, torch.from_numpy(mu).double(), torch.from_numpy(var).double(), torch.from_numpy(g).double(),
                      torch.from_numpy(be).double(), False, 0.0, 1e-5).relu()
    out.update(conv_x=x, conv_w=w, conv_g=g, conv_b=be, conv_mu=mu, conv_var=var,
               conv_y=t.permute(0, 2, 3, 1).numpy().astype(np.float32),
               conv_bn_relu=tb.permute(0, 2, 3, 1).numpy().astype(np.float32))

    # 1x1 convolution, stride 2 (ResNet downsample)
    w1 = (f32(12, 16, 1, 1) * 0.2).astype(np.float32)
    t = F.conv2d(torch.from_numpy(x).double().permute(0, 3, 1, 2), torch.from_numpy(w1).double(), stride=2)
    out.update(conv1_w=w1, conv1_y=t.permute(0, 2, 3, 1).numpy().astype(np.float32))

    # depthwise 3x3
    wd = f32(16, 1, 3, 3)
    t = F.conv2d(torch.from_numpy(x).double().permute(0, 3, 1, 2), torch.from_numpy(wd).double(), padding=1, groups=16)
    out.update(dw_w=wd, dw_y=t.permute(0, 2, 3, 1).numpy().astype(np.float32))

    # LayerNorm with residual, eps 1e-12 (BERT)
    a, r, lg, lb = f32(11, 96) * 2 + 1, f32(11, 96), f32(96), f32(96)
    t = F.layer_norm(torch.from_numpy(a + r).double(), (96,), torch.from_numpy(lg).double(), torch.from_numpy(lb).double(),
                     1e-12)
    out.update(ln_x=a, ln_r=r, ln_g=lg, ln_b=lb, ln_y=t.numpy().astype(np.float32))

    # masked softmax
    s = f32(6, 40) * 3
    m = np.where(rng.random((6, 40)) < 0.3, -1e9, 0).astype(np.float32)
    m[:, 0] = 0
    t = torch.softmax(torch.from_numpy(s).double() * 0.125 + torch.from_numpy(m).double(), -1)
    out.update(sm_x=s, sm_mask=m, sm_y=t.numpy().astype(np.float32))

    # attention, head width 64 (the fused kernel's case), with a key mask
    q, k, v = f32(2, 40, 2, 64), f32(2, 40, 2, 64), f32(2, 40, 2, 64)
    am = np.where(rng.random((2, 40)) < 0.25, -1e4, 0).astype(np.float32)
    am[:, 0] = 0
    t = F.scaled_dot_product_attention(*(torch.from_numpy(u).double().permute(0, 2, 1, 3) for u in (q, k, v)),
                                       attn_mask=torch.from_numpy(am).double()[:, None, None, :], scale=0.125)
    out.update(att_q=q, att_k=k, att_v=v, att_mask=am, att_y=t.permute(0, 2, 1, 3).numpy().astype(np.float32))

    # max pool 3x3 / 2 pad 1 and global average pool, NHWC
    t = torch.from_numpy(x).double().permute(0, 3, 1, 2)
    out.update(maxpool_y=F.max_pool2d(t, 3, 2, 1).permute(0, 2, 3, 1).numpy().astype(np.float32),
               avgpool_y=t.mean((2, 3)).numpy().astype(np.float32))

    # embedding: word + position + token type
    word, pos, typ = f32(30, 24), f32(12, 24), f32(2, 24)
    ids = rng.integers(0, 30, (2, 9)).astype(np.int64)
    tids = rng.integers(0, 2, (2, 9)).astype(np.int64)
    e = word[ids] .astype(np.float64) + pos[np.arange(9)][None].astype(np.float64) + typ[tids].astype(np.float64)
    out.update(emb_word=word, emb_pos=pos, emb_typ=typ, emb_ids=ids, emb_tids=tids,
               emb_y=e.reshape(18, 24).astype(np.float32))

    # convolution 3x3 stride 1 pad 1, 16 -> 32 channels, + residual + ReLU on the image of the first case (odd
    # height: the last row of 2x2 output tiles is half empty).  Drawn last so that every earlier vector keeps its
    # values.  The shape the Winograd path takes; the direct kernels are checked on it as well.
    ws1, rs1 = f32(32, 16, 3, 3) * np.float32(1.0 / 12.0), f32(2, 9, 8, 32)
    t = F.conv2d(torch.from_numpy(x).double().permute(0, 3, 1, 2), torch.from_numpy(ws1).double(), stride=1, padding=1)
    t = torch.relu(t.permute(0, 2, 3, 1) + torch.from_numpy(rs1).double())
    out.update(conv_s1_w=ws1, conv_s1_res=rs1, conv_s1_y=t.numpy().astype(np.float32))

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
