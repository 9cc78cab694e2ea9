"""A W8A8 OPT-shaped decoder layer assembled from the int8 modules.

Not part of the reference tree: its modules are the building blocks ("For qkv_proj", "For fc1",
"For fc2 and out_proj", nn/linear.py:19,71,126) and the layer that chains them lives in the
caller (SmoothQuant-style Int8OPTDecoderLayer).  This module is that caller for benchmarks and
end-to-end tests: every heavy step is one of the package's HIP kernels, torch only reshapes.

    hidden fp32 [B,S,H]
      LayerNormQ -> int8                                    (layer_norm_fwd_fused_single_pass_q)
      q,k,v = 3 x W8A8B8O8Linear -> int8, one launch        (linear_group_a8_w8_b8_o8)
      scores = BMM_S8T_S8N_S8T(q, k) -> int8                (bmm_s8t_s8n_s8t)
      probs  = softmax_q(scores, causal) -> int8 [0,127]    (ti_softmax_q)
      ctx    = BMM_S8T_S8N_S8T(probs, v^T) -> int8, written head-merged through output strides
               (with `fused_attention`, the default for 128 or more query positions and for 16 or fewer,
               these three run as one kernel, ti_attention_i8, and scores / probabilities never reach memory)
      acc    = W8A8B32O32LinearWithoutScaling(ctx) -> int32 (linear_a8_w8_b32_o32)   out_proj
      resid, h8 = DQ_Add_LayerNorm_Q(hidden, acc)           (ti_dq_add_layernorm_q)
      f8     = W8A8BFP32OFP32_GeLu_Q(h8) -> int8            (GEMM + GELU-quant epilogue)   fc1
      out    = W8A8BFP32OFP32Linear(f8) + resid -> fp32                                  fc2
               (one library call, ti_linear_i8_residual_f32: in decode the GEMM kernel adds the residual)
"""
from __future__ import annotations

import torch

from ..kernels.bmm import bmm_s8t_s8n_s8t
from ..kernels.fused import attention_i8, kv_append_i8, softmax_q, transpose_i8
from ..kernels.linear import linear_group_a8_w8_b8_o8, linear_qkv_decode_a8_w8_b8_o8
from .fused import DQ_Add_LayerNorm_Q, LayerNormQ, W8A8BFP32OFP32_GeLu_Q
from .linear import W8A8B8O8Linear, W8A8B32O32LinearWithoutScaling, W8A8BFP32OFP32Linear


class W8A8OPTDecoderLayer(torch.nn.Module):
    def __init__(self, hidden=5120, heads=40, ffn=20480, causal=True):
        super().__init__()
        assert hidden % heads == 0
        self.hidden, self.heads, self.head_dim, self.ffn, self.causal = hidden, heads, hidden // heads, ffn, causal
        self.ln1 = LayerNormQ(hidden)
        self.q_proj = W8A8B8O8Linear(hidden, hidden)
        self.k_proj = W8A8B8O8Linear(hidden, hidden)
        self.v_proj = W8A8B8O8Linear(hidden, hidden)
        self.out_proj = W8A8B32O32LinearWithoutScaling(hidden, hidden)
        self.ln2 = DQ_Add_LayerNorm_Q(hidden)
        self.fc1 = W8A8BFP32OFP32_GeLu_Q(hidden, ffn)
        self.fc2 = W8A8BFP32OFP32Linear(ffn, hidden)
        # attention scales: int8 scores = q8(qk_alpha * q.k), probabilities = softmax(scores * score_scale),
        # int8 context = q8(pv_alpha * P.V)
        self.qk_alpha = 1e-3
        self.score_scale = 0.05
        self.pv_alpha = 1.0 / 127.0
        # one-kernel attention for prefill-sized blocks of queries and for decode-sized ones (16 or fewer
        # rows per head); the three-launch chain in between (too few workgroups for the block kernel)
        self.fused_attention = True
        self.fused_attention_min_queries = 128
        # fc2 and the residual add that follows it as one library call (a traced forward keeps them apart
        # so that the fc2 output can be inspected)
        self.fused_residual = True

    @torch.no_grad()
    def randomize(self, seed=0):
        """Random int8 weights and per-tensor scales drawn uniformly from [1e-3, 1e-2]."""
        g = torch.Generator(device="cpu").manual_seed(seed)

        def s():
            return float(torch.empty(1).uniform_(1e-3, 1e-2, generator=g))

        for lin in (self.q_proj, self.k_proj, self.v_proj, self.out_proj, self.fc1, self.fc2):
            lin.weight = torch.randint(-127, 128, tuple(lin.weight.shape), dtype=torch.int8, generator=g).to(lin.weight.device)
        for lin in (self.q_proj, self.k_proj, self.v_proj):
            lin.bias = torch.randint(-127, 128, (self.hidden,), dtype=torch.int8, generator=g).to(lin.bias.device)
            lin.a = torch.tensor(s() / 10, dtype=torch.float32, device=lin.a.device)
            lin.b = torch.tensor(s(), dtype=torch.float32, device=lin.b.device)
        self.out_proj.bias = torch.randint(-1000, 1000, (self.hidden,), dtype=torch.int32, generator=g).to(self.out_proj.bias.device)
        self.ln2.input_scale = s() / 100
        self.fc1.bias = torch.randn(self.ffn, generator=g).to(self.fc1.bias.device)
        self.fc1.a = torch.tensor(s() / 30, dtype=torch.float32, device=self.fc1.a.device)
        self.fc1.b = torch.tensor(20.0, dtype=torch.float32, device=self.fc1.b.device)
        self.fc2.bias = torch.randn(self.hidden, generator=g).to(self.fc2.bias.device)
        self.fc2.a = torch.tensor(s() / 100, dtype=torch.float32, device=self.fc2.a.device)
        for ln in (self.ln1, self.ln2):
            ln.weight = (torch.randn(self.hidden, generator=g) * 0.1 + 1.0).div(0.05).to(ln.weight.device)
            ln.bias = (torch.randn(self.hidden, generator=g) * 0.1).div(0.05).to(ln.bias.device)
        return self

    def _qkv_pack(self):
        """The three projections' weights, biases and scales stacked for the grouped launch.  Built
        on first use and whenever one of the modules' tensors was replaced or moved; the modules'
        weight / bias are then re-pointed at slices of the pack, so the weights exist once."""
        mods = (self.q_proj, self.k_proj, self.v_proj)
        key = tuple((m.weight.data_ptr(), m.bias.data_ptr(), m.a.data_ptr(), m.b.data_ptr()) for m in mods)
        if getattr(self, "_qkv_key", None) != key:
            H = self.hidden
            w = torch.cat([m.weight for m in mods], dim=0).contiguous()
            bias = torch.cat([m.bias for m in mods], dim=0).contiguous()
            a = torch.stack([m.a.reshape(()) for m in mods]).to(torch.float32).contiguous()
            b = torch.stack([m.b.reshape(()) for m in mods]).to(torch.float32).contiguous()
            for i, m in enumerate(mods):
                m.weight, m.bias = w[i * H:(i + 1) * H], bias[i * H:(i + 1) * H]
                m.a, m.b = a[i], b[i]
            self._qkv = (w, bias, a, b)
            self._qkv_key = tuple((m.weight.data_ptr(), m.bias.data_ptr(), m.a.data_ptr(), m.b.data_ptr()) for m in mods)
        return self._qkv

    def _heads(self, t, B, S):
        # [B,S,H] int8 -> [B*heads, S, D].  One batch: a strided view (the BMM takes row and batch
        # strides, each head's rows stay K-contiguous).  Several batches: a copy.
        if B == 1:
            return t.view(S, self.heads, self.head_dim).transpose(0, 1)
        return t.view(B, S, self.heads, self.head_dim).transpose(1, 2).reshape(B * self.heads, S, self.head_dim)

    @torch.no_grad()
    def forward(self, hidden, kv_cache=None, _trace=None, _mark=None):
        """hidden fp32 [B,S,H].  kv_cache = (K int8 [B*heads, T, D], V^T int8 [B*heads, D, T]) holds the
        T-S earlier positions in its first T-S slots; the S new positions are written into the last S
        slots before attention (decode / chunked prefill).  Returns fp32 [B,S,H].  A dict passed as
        `_trace` receives every intermediate tensor (for stage-by-stage parity tests); a callable
        passed as `_mark` is called with a stage name after that stage's launches (for timing the
        stages in sequence with stream events)."""
        mark = _mark if _mark is not None else (lambda name: None)
        B, S, H = hidden.shape
        h8 = self.ln1(hidden)
        mark("ln1_layernorm_q")
        w3, b3, a3, s3 = self._qkv_pack()
        qkv = None
        if kv_cache is not None and B == 1 and S <= 16:
            # decode: projections and KV-cache append in one launch
            qkv = linear_qkv_decode_a8_w8_b8_o8(h8.view(S, H), w3, b3, a3, s3, kv_cache[0], kv_cache[1])
        appended = qkv is not None
        if appended:
            qkv = qkv.view(1, S, 3 * H)
        else:
            qkv = linear_group_a8_w8_b8_o8(h8, w3, b3, a3, s3, 3)                   # [B,S,3H] int8
        q = self._heads(qkv[..., :H], B, S)
        k_new = self._heads(qkv[..., H:2 * H], B, S)
        v = qkv[..., 2 * H:]                                                       # [B,S,H] int8, row pitch 3H
        mark("qkv_3x_linear_o8")
        if kv_cache is None:
            k_all = k_new
            vt_all = torch.empty((B * self.heads, self.head_dim, S), dtype=torch.int8, device=hidden.device)
            # V^T of every head of a batch in one transpose: [S, heads*D] -> [heads*D, S]
            for b in range(B):
                transpose_i8(v[b], out=vt_all[b * self.heads:(b + 1) * self.heads].view(H, S))
        else:
            # the new K rows and V^T columns go into the last S slots of the cache, one launch per batch
            k_all, vt_all = kv_cache
            if appended:
                pass
            elif k_all.is_contiguous() and vt_all.is_contiguous() and self.head_dim % 16 == 0:
                for b in range(B):
                    hs = slice(b * self.heads, (b + 1) * self.heads)
                    kv_append_i8(qkv[b, :, H:2 * H], v[b], k_all[hs], vt_all[hs])
            else:
                T = k_all.shape[1]
                k_all[:, T - S:, :] = k_new
                for b in range(B):
                    transpose_i8(v[b], out=vt_all[b * self.heads:(b + 1) * self.heads].view(H, T)[:, T - S:])
        mark("kv_append_v_transpose")
        T = k_all.shape[1]
        ctx = torch.empty((B, S, H), dtype=torch.int8, device=hidden.device)
        # 16 or fewer query rows (decode) against up to 4096 keys run the kernel's one-workgroup-per-head form
        fused = (self.fused_attention and (S >= self.fused_attention_min_queries or (S <= 16 and T <= 4096))
                 and self.head_dim == 128 and T % 16 == 0 and self.score_scale > 0.0)
        scores = probs = None
        if fused:
            for b in range(B):
                hs = slice(b * self.heads, (b + 1) * self.heads)
                attention_i8(q[hs], k_all[hs], vt_all[hs], self.qk_alpha, self.score_scale, self.pv_alpha,
                             causal_q_len=S if self.causal else 0,
                             out=ctx[b].view(S, self.heads, self.head_dim).transpose(0, 1))
            mark("attention_i8_fused")
        else:
            scores = bmm_s8t_s8n_s8t(q, k_all, self.qk_alpha)                       # [B*heads, S, T] int8
            mark("qk_bmm_o8")
            probs = softmax_q(scores, self.score_scale, causal_q_len=S if self.causal else 0)
            mark("softmax_q")
            # P.V with the head merge folded into the output strides: head h of batch b writes columns
            # h*D .. h*D+D of row (b, s) of a [B,S,H] tensor
            for b in range(B):
                out_view = ctx[b].view(S, self.heads, self.head_dim).transpose(0, 1)   # [heads, S, D] strided
                bmm_s8t_s8n_s8t(probs[b * self.heads:(b + 1) * self.heads], vt_all[b * self.heads:(b + 1) * self.heads],
                                self.pv_alpha, out=out_view)
            mark("pv_bmm_o8")
        acc = self.out_proj(ctx)                                                    # int32 [B,S,H]
        mark("out_proj_linear_o32")
        resid, h8b = self.ln2(hidden, acc)
        mark("ln2_dq_add_layernorm_q")
        f8 = self.fc1(h8b)
        mark("fc1_linear_gelu_q")
        if self.fused_residual and _trace is None:
            y = None
            out = self.fc2.forward_add(f8, resid)   # one launch: the GEMM kernel adds the residual as it stores
            mark("fc2_linear_f32_plus_residual")
        else:
            y = self.fc2(f8)
            mark("fc2_linear_f32")
            out = y + resid
            mark("residual_add")
        if _trace is not None:
            _trace.update(h8=h8, q=q, k_all=k_all, vt_all=vt_all, scores=scores, probs=probs, ctx=ctx, acc=acc,
                          resid=resid, h8b=h8b, f8=f8, fc2=y, out=out)
        return out
