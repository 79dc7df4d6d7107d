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


def init_weights(arch="bert-base", seed=0, vocab=30522, max_pos=512, type_vocab=2, cfg=None, qa_head=False):
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
    if qa_head:
        # BertForQuestionAnswering (what the reference serves, tests/endpoint.py:36-40): span start / end logits
        linear("qa_outputs", 2, H)
    return w


class Bert(Function):
    """inputs: ids [B, S] int64, then token type ids [B, S] int64 if `token_types`, then the
    attention mask [B, S] (1 = attend, 0 = padding) if `masked`.  Outputs: last hidden state and
    pooled output, or, with a `qa_outputs` head in the weights, the span start and end logits
    [B, S] each (transformers.BertForQuestionAnswering)."""

    def __init__(self, server, fid, arch="bert-base", batch=1, seq=128, weights=None, seed=0, level=1, cfg=None,
                 vocab=30522, token_types=False, masked=False):
        super().__init__(server, fid, level)
        self.token_types, self.masked = token_types, masked
        self.cfg = dict(CONFIGS[arch]) if cfg is None else dict(cfg)
        self.batch, self.seq = batch, seq
        self._weights = weights if weights is not None else init_weights(arch, seed, vocab=vocab, cfg=self.cfg)
        self.vocab = self._weights["embeddings.word_embeddings.weight"].shape[0]
        self.max_pos = self._weights["embeddings.position_embeddings.weight"].shape[0]
        self.type_vocab = self._weights["embeddings.token_type_embeddings.weight"].shape[0]
        self.qa_head = "qa_outputs.weight" in self._weights

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
        specs = [((self.batch, self.seq), np.int64)]
        if self.token_types:
            specs.append(((self.batch, self.seq), np.int64))
        if self.masked:
            specs.append(((self.batch, self.seq), np.float32))   # additive form, see additive_mask()
        return specs

    @staticmethod
    def additive_mask(attention_mask):
        """1 / 0 attention mask -> the additive float mask the model adds to the scores
        (0 where attended, the most negative float32 where not: transformers' convention)."""
        m = np.asarray(attention_mask, dtype=np.float32)
        return ((1.0 - m) * np.finfo(np.float32).min).astype(np.float32)

    def _linear(self, x, tok, inp, out, name, act=ACT_NONE, xs_r=None):
        y = self.alloc(tok * out * 4)
        self.s.gemm(self.fid, x.va, self.w[name + ".weight"], y.va, tok, out, inp,
                    xs_r=inp if xs_r is None else xs_r, ys_c=inp, ldc=out, bias=self.w[name + ".bias"], act=act)
        return y

    def _ln(self, x, res, tok, name, dst=None):
        H = self.cfg["hidden"]
        y = self.alloc(tok * H * 4) if dst is None else dst
        self.s.launch(self.fid, OP_LAYERNORM,
                      [x.va, res.va if res is not None else 0, self.w[name + ".weight"], self.w[name + ".bias"], y.va],
                      [tok, H], [LN_EPS])
        return y

    def forward(self, inputs):
        ids = inputs[0]
        tt_va = inputs[1].va if self.token_types else 0
        mask_va = inputs[-1].va if self.masked else 0
        B, S = self.batch, self.seq
        H, A, F, L = self.cfg["hidden"], self.cfg["heads"], self.cfg["ffn"], self.cfg["layers"]
        dh = H // A
        tok = B * S
        emb = self.alloc(tok * H * 4)
        self.s.launch(self.fid, OP_EMBEDDING,
                      [ids.va, tt_va, self.w["embeddings.word_embeddings.weight"],
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
                self.s.launch(self.fid, OP_ATTENTION, [q_va, k_va, v_va, mask_va, ctx.va],
                              [B, A, S, dh, H3, H3, H3, H], [scale])
            else:
                scores = self.alloc(B * A * S * S * 4)
                # scores[b,a] = Q[b,:,a,:] . K[b,:,a,:]^T
                self.s.gemm(self.fid, q_va, k_va, scores.va, S, S, dh, xs_r=H3, ys_c=H3, ldc=S, nb0=B, nb1=A,
                            xb0=S * H3, xb1=dh, yb0=S * H3, yb1=dh, cb0=A * S * S, cb1=S * S)
                probs = self.alloc(B * A * S * S * 4)
                self.s.launch(self.fid, OP_SOFTMAX, [scores.va, mask_va, probs.va], [B * A * S, S, A * S], [scale])
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
            # One result buffer = [last hidden state | pooled], because the first D2H copy of a request is its
            # completion marker (reference cuda_server.hpp:1044): the last LayerNorm writes straight into it.
            result = self.alloc((tok * H + B * H) * 4) if (i == L - 1 and not self.qa_head) else None
            h = self._ln(out, h1, tok, p + ".output.LayerNorm", dst=result)
            self.release(out)
            self.release(h1)
        if self.qa_head:
            # span logits [tok, 2]; de-interleaved into start / end on the host
            out = self._linear(h, tok, H, 2, "qa_outputs")
            self.release(h)
            return [(out, (tok * 2,), np.float32)]
        if L == 0:      # no encoder layer: the embedding output is the last hidden state
            result = self.alloc((tok * H + B * H) * 4)
            self.s.d2d(self.fid, result.va, h.va, tok * H * 4)
            self.release(h)
            h = result
        # pooler: tanh(W . h[:, 0] + b); row b of X is token b*S
        self.s.gemm(self.fid, h.va, self.w["pooler.dense.weight"], h.va + tok * H * 4, B, H, H,
                    xs_r=S * H, ys_c=H, ldc=H, bias=self.w["pooler.dense.bias"], act=ACT_TANH)
        return [(h, (tok * H + B * H,), np.float32)]

    def postprocess(self, host):
        (flat,) = host
        B, S, H = self.batch, self.seq, self.cfg["hidden"]
        if self.qa_head:
            logits = flat.reshape(B, S, 2)
            return [np.ascontiguousarray(logits[..., 0]), np.ascontiguousarray(logits[..., 1])]
        return [flat[:B * S * H].reshape(B, S, H), flat[B * S * H:].reshape(B, H)]
