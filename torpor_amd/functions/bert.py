"""BERT-base / BERT-large encoder (+ pooler) as a served function.

The reference serves Hugging Face BERT models (tests/endpoint.py:37-60); their Linear layers
reach the server as cublasSgemm, the attention products as cublasSgemmStridedBatched and
everything else as libtorch kernel launches.  Here: dense GEMMs with bias (+GELU / tanh) fused in
the epilogue, the query / key / value projections as one GEMM over the stacked [3H, H] weight
(stacked once, at upload; 4.5 tiles per CU instead of three launches of 1.5), head-strided
the attention core as one fused kernel reading the heads in place from that [tokens, 3H]
projection (head width 64; other widths fall back to two head-strided batched GEMMs around a
softmax launch), and residual LayerNorm.  Weight names
and conventions follow `transformers.BertModel` (LayerNorm eps 1e-12, erf GELU, additive mask,
absolute position + token-type embeddings, tanh pooler on the first token).
"""
from collections import OrderedDict

import numpy as np

from ..server import ACT_GELU, ACT_NONE, ACT_TANH, OP_ATTENTION, OP_EMBEDDING, OP_LAYERNORM, OP_SOFTMAX
from .base import Function

CONFIGS = {
    "bert-base": dict(layers=12, hidden=768, heads=12, ffn=3072),
    "bert-large": dict(layers=24, hidden=1024, heads=16, ffn=4096),
}
LN_EPS = 1e-12


def init_weights(arch="bert-base", seed=0, vocab=30522, max_pos=512, type_vocab=2, cfg=None):
    """Random-init weights: N(0, 0.02) matrices, embeddings and biases, LayerNorm gamma
    N(1, 0.02) / beta N(0, 0.02).  (Hugging Face zero-initialises biases and uses gamma=1,
    beta=0; small random values are used instead so that every tensor influences the output.)"""
    import torch

    c = dict(CONFIGS[arch]) if cfg is None else dict(cfg)
    H, F, L = c["hidden"], c["ffn"], c["layers"]
    g = torch.Generator().manual_seed(seed)
    w = OrderedDict()

    def normal(name, *shape, mean=0.0):
        w[name] = torch.empty(*shape).normal_(mean, 0.02, generator=g).numpy()

    def linear(name, out, inp):
        normal(name + ".weight", out, inp)
        normal(name + ".bias", out)

    def ln(name):
        normal(name + ".weight", H, mean=1.0)
        normal(name + ".bias", H)

    normal("embeddings.word_embeddings.weight", vocab, H)
    normal("embeddings.position_embeddings.weight", max_pos, H)
    normal("embeddings.token_type_embeddings.weight", type_vocab, H)
    ln("embeddings.LayerNorm")
    for i in range(L):
        p = f"encoder.layer.{i}"
        linear(p + ".attention.self.query", H, H)
        linear(p + ".attention.self.key", H, H)
        linear(p + ".attention.self.value", H, H)
        linear(p + ".attention.output.dense", H, H)
        ln(p + ".attention.output.LayerNorm")
        linear(p + ".intermediate.dense", F, H)
        linear(p + ".output.dense", H, F)
        ln(p + ".output.LayerNorm")
    linear("pooler.dense", H, H)
    return w


class Bert(Function):
    def __init__(self, server, fid, arch="bert-base", batch=1, seq=128, weights=None, seed=0, level=1, cfg=None,
                 vocab=30522):
        super().__init__(server, fid, level)
        self.cfg = dict(CONFIGS[arch]) if cfg is None else dict(cfg)
        self.batch, self.seq = batch, seq
        self._weights = weights if weights is not None else init_weights(arch, seed, vocab=vocab, cfg=self.cfg)
        self.vocab = self._weights["embeddings.word_embeddings.weight"].shape[0]
        self.max_pos = self._weights["embeddings.position_embeddings.weight"].shape[0]
        self.type_vocab = self._weights["embeddings.token_type_embeddings.weight"].shape[0]

    def weights(self):
        """Tensors as uploaded: the Hugging Face state dict, except that each layer's query, key
        and value matrices (and biases) are stacked into `attention.self.qkv.{weight,bias}`."""
        out = OrderedDict()
        for k, v in self._weights.items():
            if ".attention.self.key." in k or ".attention.self.value." in k:
                continue
            if ".attention.self.query." in k:
                parts = [self._weights[k.replace(".query.", f".{n}.")] for n in ("query", "key", "value")]
                out[k.replace(".query.", ".qkv.")] = np.ascontiguousarray(np.concatenate(parts, axis=0), dtype=np.float32)
            else:
                out[k] = np.ascontiguousarray(v, dtype=np.float32)
        return out

    def input_specs(self):
        return [((self.batch, self.seq), np.int64)]

    def _linear(self, x, tok, inp, out, name, act=ACT_NONE, xs_r=None):
        y = self.alloc(tok * out * 4)
        self.s.gemm(self.fid, x.va, self.w[name + ".weight"], y.va, tok, out, inp,
                    xs_r=inp if xs_r is None else xs_r, ys_c=inp, ldc=out, bias=self.w[name + ".bias"], act=act)
        return y

    def _ln(self, x, res, tok, name):
        H = self.cfg["hidden"]
        y = self.alloc(tok * H * 4)
        self.s.launch(self.fid, OP_LAYERNORM,
                      [x.va, res.va if res is not None else 0, self.w[name + ".weight"], self.w[name + ".bias"], y.va],
                      [tok, H], [LN_EPS])
        return y

    def forward(self, inputs):
        (ids,) = inputs
        B, S = self.batch, self.seq
        H, A, F, L = self.cfg["hidden"], self.cfg["heads"], self.cfg["ffn"], self.cfg["layers"]
        dh = H // A
        tok = B * S
        emb = self.alloc(tok * H * 4)
        self.s.launch(self.fid, OP_EMBEDDING,
                      [ids.va, 0, self.w["embeddings.word_embeddings.weight"],
                       self.w["embeddings.position_embeddings.weight"],
                       self.w["embeddings.token_type_embeddings.weight"], emb.va],
                      [tok, S, H, self.vocab, self.type_vocab])
        h = self._ln(emb, None, tok, "embeddings.LayerNorm")
        self.release(emb)
        scale = 1.0 / float(np.sqrt(dh))
        for i in range(L):
            p = f"encoder.layer.{i}"
            # row t of qkv = [Q | K | V] of token t
            qkv = self._linear(h, tok, H, 3 * H, p + ".attention.self.qkv")
            H3 = 3 * H
            q_va, k_va, v_va = qkv.va, qkv.va + H * 4, qkv.va + 2 * H * 4
            ctx = self.alloc(tok * H * 4)
            if dh == 64:
                # fused softmax(Q.K^T / sqrt(dh)) . V, heads read in place from the [tok, 3H] projection
                self.s.launch(self.fid, OP_ATTENTION, [q_va, k_va, v_va, 0, ctx.va],
                              [B, A, S, dh, H3, H3, H3, H], [scale])
            else:
                scores = self.alloc(B * A * S * S * 4)
                # scores[b,a] = Q[b,:,a,:] . K[b,:,a,:]^T
                self.s.gemm(self.fid, q_va, k_va, scores.va, S, S, dh, xs_r=H3, ys_c=H3, ldc=S, nb0=B, nb1=A,
                            xb0=S * H3, xb1=dh, yb0=S * H3, yb1=dh, cb0=A * S * S, cb1=S * S)
                probs = self.alloc(B * A * S * S * 4)
                self.s.launch(self.fid, OP_SOFTMAX, [scores.va, 0, probs.va], [B * A * S, S, A * S], [scale])
                self.release(scores)
                # ctx[b,:,a,:] = P[b,a] . V[b,:,a,:]
                self.s.gemm(self.fid, probs.va, v_va, ctx.va, S, dh, S, xs_r=S, ys_c=1, ys_k=H3, ldc=H, nb0=B, nb1=A,
                            xb0=A * S * S, xb1=S * S, yb0=S * H3, yb1=dh, cb0=S * H, cb1=dh)
                self.release(probs)
            self.release(qkv)
            ao = self._linear(ctx, tok, H, H, p + ".attention.output.dense")
            self.release(ctx)
            h1 = self._ln(ao, h, tok, p + ".attention.output.LayerNorm")
            self.release(ao)
            self.release(h)
            inter = self._linear(h1, tok, H, F, p + ".intermediate.dense", act=ACT_GELU)
            out = self._linear(inter, tok, F, H, p + ".output.dense")
            self.release(inter)
            h = self._ln(out, h1, tok, p + ".output.LayerNorm")
            self.release(out)
            self.release(h1)
        # One result buffer = [last hidden state | pooled], because the first D2H copy of a request
        # is its completion marker (reference cuda_server.hpp:1044).
        out = self.alloc((tok * H + B * H) * 4)
        self.s.d2d(self.fid, out.va, h.va, tok * H * 4)
        # pooler: tanh(W . h[:, 0] + b); row b of X is token b*S
        self.s.gemm(self.fid, h.va, self.w["pooler.dense.weight"], out.va + tok * H * 4, B, H, H,
                    xs_r=S * H, ys_c=H, ldc=H, bias=self.w["pooler.dense.bias"], act=ACT_TANH)
        self.release(h)
        return [(out, (tok * H + B * H,), np.float32)]

    def postprocess(self, host):
        (flat,) = host
        B, S, H = self.batch, self.seq, self.cfg["hidden"]
        return [flat[:B * S * H].reshape(B, S, H), flat[B * S * H:].reshape(B, H)]
