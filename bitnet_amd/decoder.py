"""BitNet-b1.58-2B-shaped decoder on top of the BitLinear library: the caller
of the hot path (gpu/model.py:87-296 and the decode loop of
gpu/generate.py:159-213, 217-304 of the reference): the model, the captured
prompt pass and decode step, and the generation loop on token ids.

Same module tree and parameter names as the reference (``layers.N.attention.
{wqkv,wo,attn_sub_norm}``, ``layers.N.feed_forward.{w13,w2,ffn_sub_norm}``,
``attention_norm``, ``ffn_norm``, ``tok_embeddings``, ``norm``, ``output``), so a
``model_state_int2.pt`` state dict loads with strict=True.  Where the reference
leans on xformers (RMSNorm, rope_padded, flash attention on a padded KV cache),
plain torch ops are used: RMSNorm and RoPE are closed forms, attention is
softmax(QK^T/sqrt(d))V in fp32 over the cache.  One decode step is captured in
a HIP graph and replayed per token, as the reference does with CUDA graphs.
"""
import time
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
from torch import nn

from . import _lib
from .bitlinear import BitLinearKernel, _ptr, _stream_ptr


@dataclass
class ModelArgs:
    # gpu/model.py:39-49
    dim: int = 2560
    n_layers: int = 30
    n_heads: int = 20
    n_kv_heads: int = 5
    vocab_size: int = 128256
    ffn_dim: int = 6912
    norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    # not in the reference: give every row of the fused wqkv / w13 products the scale of the sub-tensor it
    # came from (what convert_checkpoint.py:42-50 stores) instead of the reference kernel's equal slots
    segment_scales: bool = False


class RMSNorm(nn.Module):
    """y = x * rsqrt(mean(x^2) + eps) * weight, evaluated in fp32 and rounded
    to the input dtype once."""

    def __init__(self, dim: int, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim), requires_grad=False)

    def forward(self, x):
        xf = x.float()
        rstd = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + self.eps)
        return (xf * rstd * self.weight.float()).to(x.dtype)


def rope_tables(head_dim: int, max_seq: int, theta: float, device) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos / sin [max_seq, head_dim // 2] in fp32 for rotation of adjacent pairs."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, device=device, dtype=torch.float32) / head_dim))
    ang = torch.outer(torch.arange(max_seq, device=device, dtype=torch.float32), inv)
    return torch.cos(ang), torch.sin(ang)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [..., n_heads, head_dim]; cos/sin broadcastable to [..., 1, head_dim/2].
    Pairs (x[2i], x[2i+1]) are rotated by the angle of frequency i, in fp32."""
    xf = x.float().unflatten(-1, (-1, 2))
    a, b = xf[..., 0], xf[..., 1]
    out = torch.stack((a * cos - b * sin, a * sin + b * cos), dim=-1)
    return out.flatten(-2).to(x.dtype)


class AttnWorkspace:
    """Scratch of the split attention kernel: tagged partial results of the
    splits (zero before the first use) and one arrival counter per (sequence,
    kv head) for the earlier kernel.  One instance
    serves all layers of a decoder (their kernels run one after the other)."""

    def __init__(self, batch: int, n_heads: int, n_kv_heads: int, n_splits: int, device):
        lib = _lib.load_library()
        self.batch = batch
        self.n_heads = n_heads
        self.n_kv_heads = n_kv_heads
        self.n_splits = n_splits
        n = lib.bitnet_attn_decode_workspace_floats(batch, n_heads, n_kv_heads, n_splits)
        if n < 0:
            raise ValueError("AttnWorkspace: bad batch / head counts / number of splits")
        self.error_index = lib.bitnet_attn_decode_error_index(batch, n_heads, n_kv_heads, n_splits)
        self.partials = torch.zeros(n, dtype=torch.float32, device=device)  # zero once: see bitnet_attn_decode
        self.counters = torch.zeros(batch * n_kv_heads, dtype=torch.int32, device=device)

    def error(self) -> int:
        """The workspace's error word (synchronises): non-zero once a merge of
        the splits' records gave up, which also left NaN rows in that call's
        output (bitnet_attn_decode_error_index)."""
        return int(self.partials[self.error_index : self.error_index + 1].view(torch.int32).item())

    def reset(self) -> None:
        """Back to the state of a fresh workspace (zero records, epochs and error word).  Not inside a graph
        capture; graphs captured on this workspace keep working, since they hold its buffers, not their contents."""
        self.partials.zero_()
        self.counters.zero_()

    def check(self) -> None:
        """Raises if a merge gave up since the last check, and clears the condition: one failed call is reported
        once and does not poison the object (later calls compute healthy results again)."""
        if self.error():
            self.reset()
            raise _lib.BitLinearLibraryError(
                "attention decode: a merge of the split records gave up (workspace not zeroed before its first use, "
                "or shared between overlapping calls); the affected output rows are NaN"
            )


def decode_step_begin(tokens, positions, emb_weight, cos, sin):
    """Embedding rows of the step's input tokens and the cos | sin rows of their
    positions in one launch (bitnet_decode_step_begin).  tokens / positions
    int64 [B]; returns (h bf16 [B, dim], rope_rows fp32 [B, 128])."""
    B = tokens.shape[0]
    V, dim = emb_weight.shape
    h = torch.empty(B, dim, dtype=torch.bfloat16, device=tokens.device)
    rows = torch.empty(B, 2 * cos.shape[1], dtype=torch.float32, device=tokens.device)
    st = _lib.load_library().bitnet_decode_step_begin(
        _ptr(tokens), _ptr(positions), _ptr(emb_weight), _ptr(cos), _ptr(sin), _ptr(h), _ptr(rows),
        B, V, dim, cos.shape[0], 2 * cos.shape[1], _stream_ptr())
    if st != 0:
        raise _lib.BitLinearLibraryError(f"bitnet_decode_step_begin: status {st}")
    return h, rows


def attn_decode(xqkv, cache_k, cache_v, positions, cos, sin, n_heads, n_kv_heads, workspace: "AttnWorkspace" = None,
                rope_rows=None):
    """Rope + KV-cache write + grouped-query attention of one new token per
    sequence in one HIP kernel (bitnet_attn_decode; bitnet_attn_decode_rows
    when the positions' cos | sin rows are handed over).  xqkv bf16 [B,
    (n_heads + 2 n_kv) * 128]; positions int64 [B]; returns bf16 [B, n_heads * 128]."""
    B = xqkv.shape[0]
    S = cache_k.shape[1]
    hd = cache_k.shape[-1]
    # the kernels index every buffer with these sizes: check them here, before any launch
    if xqkv.dtype != torch.bfloat16 or cache_k.dtype != torch.bfloat16 or cache_v.dtype != torch.bfloat16:
        raise TypeError("attn_decode: xqkv and the caches must be bfloat16")
    if xqkv.shape != (B, (n_heads + 2 * n_kv_heads) * hd):
        raise ValueError(f"attn_decode: xqkv has shape {tuple(xqkv.shape)}, expected {(B, (n_heads + 2 * n_kv_heads) * hd)}")
    if cache_k.shape != (B, S, n_kv_heads, hd) or cache_v.shape != cache_k.shape:
        raise ValueError("attn_decode: the caches must be [batch, max_seq, n_kv_heads, head_dim] with the batch of xqkv")
    if positions.dtype != torch.int64 or positions.numel() != B:
        raise ValueError("attn_decode: positions must be int64 [batch]")
    if cos.shape[0] < S or sin.shape[0] < S:
        raise ValueError("attn_decode: the rope tables have fewer rows than the cache has positions")
    if workspace is not None and (workspace.batch != B or workspace.n_heads != n_heads or workspace.n_kv_heads != n_kv_heads):
        raise ValueError("attn_decode: the workspace was sized for another batch or head count")
    if rope_rows is not None and (rope_rows.dtype != torch.float32 or rope_rows.shape != (B, hd)):
        raise ValueError("attn_decode: rope_rows must be float32 [batch, head_dim]")
    out = torch.empty(B, n_heads * hd, dtype=torch.bfloat16, device=xqkv.device)
    ns = workspace.n_splits if workspace is not None else 1
    lib = _lib.load_library()
    wsp = _ptr(workspace.partials) if workspace is not None else None
    wsc = _ptr(workspace.counters) if workspace is not None else None
    if rope_rows is not None:
        st = lib.bitnet_attn_decode_rows(
            _ptr(xqkv), _ptr(cache_k), _ptr(cache_v), _ptr(positions), _ptr(cos), _ptr(sin), _ptr(rope_rows), _ptr(out),
            wsp, wsc, ns, B, S, n_heads, n_kv_heads, hd, _stream_ptr())
    else:
        st = lib.bitnet_attn_decode(
            _ptr(xqkv), _ptr(cache_k), _ptr(cache_v), _ptr(positions), _ptr(cos), _ptr(sin), _ptr(out),
            wsp, wsc, ns, B, S, n_heads, n_kv_heads, hd, _stream_ptr())
    if st != 0:
        raise _lib.BitLinearLibraryError(f"bitnet_attn_decode: status {st}")
    return out


def rope_cache_tokens(xqkv, cache_k, cache_v, positions, cos, sin, n_heads, n_kv_heads):
    """Rope + KV-cache write for T new tokens per sequence in one HIP kernel
    (bitnet_rope_cache_tokens).  xqkv bf16 [B * T, (n_heads + 2 n_kv) * 128];
    positions int64 [B, T]; returns the rotated q, bf16 [B, T, n_heads, 128]."""
    B, T = positions.shape
    S = cache_k.shape[1]
    hd = cache_k.shape[-1]
    q = torch.empty(B, T, n_heads, hd, dtype=torch.bfloat16, device=xqkv.device)
    st = _lib.load_library().bitnet_rope_cache_tokens(
        _ptr(xqkv), _ptr(cache_k), _ptr(cache_v), _ptr(positions), _ptr(cos), _ptr(sin), _ptr(q),
        B, T, S, n_heads, n_kv_heads, hd, _stream_ptr(),
    )
    if st != 0:
        raise _lib.BitLinearLibraryError(f"bitnet_rope_cache_tokens: status {st}")
    return q


def attn_prefill(q, cache_k, cache_v, start: int = 0):
    """Causal grouped-query attention of T new tokens per sequence over cache
    rows 0 .. start + t in one HIP kernel (bitnet_attn_prefill).  q bf16
    [B, T, n_heads, 128] (rotated); returns bf16 [B * T, n_heads * 128]."""
    B, T, n_heads, hd = q.shape
    S, n_kv = cache_k.shape[1], cache_k.shape[2]
    out = torch.empty(B * T, n_heads * hd, dtype=torch.bfloat16, device=q.device)
    st = _lib.load_library().bitnet_attn_prefill(
        _ptr(q), _ptr(cache_k), _ptr(cache_v), _ptr(out), B, T, S, start, n_heads, n_kv, hd, _stream_ptr())
    if st != 0:
        raise _lib.BitLinearLibraryError(f"bitnet_attn_prefill: status {st}")
    return out


class LmHeadWorkspace:
    """Scratch of bitnet_lm_head_greedy for one (batch, vocabulary, dim)."""

    def __init__(self, batch: int, vocab: int, dim: int, device):
        lib = _lib.load_library()
        n = lib.bitnet_lm_head_workgroups(vocab) * 16
        self.y = torch.empty(batch, dim, dtype=torch.bfloat16, device=device)
        self.part_val = torch.empty(n, dtype=torch.float32, device=device)
        self.part_idx = torch.empty(n, dtype=torch.int32, device=device)


def lm_head_greedy(h, norm: "RMSNorm", emb_weight, workspace: LmHeadWorkspace, token_out=None, logits_out=None,
                   next_input=None, positions=None, history=None, step_idx=None):
    """Final RMSNorm + tied bf16 LM head + greedy token in three launches
    (bitnet_lm_head_greedy).  h bf16 [B, dim]; returns int64 [B] (token_out if
    given); logits_out fp32 [B, vocab] receives the bf16-rounded logits if given.
    With next_input / positions / history + step_idx (int64 device tensors) the
    last launch also does a decode step's bookkeeping: next_input = token,
    positions += 1, history[step_idx[0]] = token, step_idx += 1."""
    B, K = h.shape
    V = emb_weight.shape[0]
    if token_out is None:
        token_out = torch.empty(B, dtype=torch.int64, device=h.device)
    opt = lambda t: _ptr(t) if t is not None else None
    st = _lib.load_library().bitnet_lm_head_greedy_step(
        _ptr(h), _ptr(norm.weight), norm.eps, _ptr(emb_weight), _ptr(workspace.y), opt(logits_out), _ptr(token_out),
        _ptr(workspace.part_val), _ptr(workspace.part_idx), opt(next_input), opt(positions), opt(history), opt(step_idx),
        B, V, K, _stream_ptr(),
    )
    if st != 0:
        raise _lib.BitLinearLibraryError(f"bitnet_lm_head_greedy_step: status {st}")
    return token_out


def norm_bitlinear(x, norm: "RMSNorm", lin: BitLinearKernel, glu: bool = False, residual=None):
    """[squared-ReLU gate ->] RMSNorm -> BitLinearKernel.forward [-> + residual]
    through bitlinear_norm_forward_bf16: one kernel for small activation blocks,
    a norm/quantizer kernel plus the product kernel for larger ones; x bf16
    [M, K] (or [M, 2K] with glu)."""
    M = x.shape[0]
    K = lin.in_features
    if x.dtype != torch.bfloat16 or not x.is_cuda or not x.is_contiguous():
        raise ValueError("norm_bitlinear: x must be a contiguous bfloat16 GPU tensor")
    if x.dim() != 2 or x.shape[1] != (2 * K if glu else K):
        raise ValueError(f"norm_bitlinear: x has shape {tuple(x.shape)}, expected [M, {2 * K if glu else K}]")
    if norm.weight.dtype != torch.bfloat16 or norm.weight.numel() != K:
        raise ValueError("norm_bitlinear: the norm weight must be bfloat16 [K]")
    if residual is not None and (residual.dtype != torch.bfloat16 or residual.shape != (M, lin.out_features)
                                 or not residual.is_contiguous()):
        raise ValueError("norm_bitlinear: residual must be contiguous bfloat16 [M, N]")
    out = torch.empty(M, lin.out_features, dtype=torch.bfloat16, device=x.device)
    q_ws = torch.empty(M, K, dtype=torch.int8, device=x.device)
    s_ws = torch.empty(M, dtype=torch.bfloat16, device=x.device)
    if lin.seg_ends is not None:
        st = _lib.load_library().bitlinear_norm_forward_bf16_seg(
            _ptr(x), _ptr(norm.weight), norm.eps, 1 if glu else 0, _ptr(lin.weight), _ptr(lin.weight_scale),
            lin._seg_c, len(lin.seg_ends), _ptr(residual) if residual is not None else None, _ptr(out), _ptr(q_ws),
            _ptr(s_ws), M, lin.out_features, K, lin.quant_mode, _stream_ptr(),
        )
        _lib.check(st, f"bitlinear_norm_forward_bf16_seg(M={M}, N={lin.out_features}, K={lin.in_features})")
        return out
    st = _lib.load_library().bitlinear_norm_forward_bf16(
        _ptr(x), _ptr(norm.weight), norm.eps, 1 if glu else 0, _ptr(lin.weight), _ptr(lin.weight_scale),
        _ptr(residual) if residual is not None else None, _ptr(out), _ptr(q_ws), _ptr(s_ws), M, lin.out_features, K,
        lin.quant_mode, _stream_ptr(),
    )
    _lib.check(st, f"bitlinear_norm_forward_bf16(M={M}, N={lin.out_features}, K={lin.in_features})")
    return out


class Attention(nn.Module):
    def __init__(self, args: ModelArgs):
        super().__init__()
        self.head_dim = args.dim // args.n_heads
        self.n_heads = args.n_heads
        self.n_kv_heads = args.n_kv_heads
        nq, nk = args.n_heads * self.head_dim, args.n_kv_heads * self.head_dim
        self.wqkv = BitLinearKernel(args.dim, nq + 2 * nk, seg_ends=(nq, nq + nk, nq + 2 * nk) if args.segment_scales else None)
        self.wo = BitLinearKernel(args.n_heads * self.head_dim, args.dim)
        self.attn_sub_norm = RMSNorm(args.dim, args.norm_eps)

    def split_qkv(self, xqkv):
        nq = self.n_heads * self.head_dim
        nk = self.n_kv_heads * self.head_dim
        q = xqkv[..., :nq].unflatten(-1, (self.n_heads, self.head_dim))
        k = xqkv[..., nq : nq + nk].unflatten(-1, (self.n_kv_heads, self.head_dim))
        v = xqkv[..., nq + nk :].unflatten(-1, (self.n_kv_heads, self.head_dim))
        return q, k, v

    def attend(self, q, keys, values, mask):
        """q [B, T, n_heads, d]; keys/values [B, S, n_kv, d]; mask [B, T, S] bool
        (True = visible).  fp32 softmax(QK^T / sqrt(d)) V with grouped heads."""
        B, T = q.shape[0], q.shape[1]
        g = self.n_heads // self.n_kv_heads
        qf = q.float().view(B, T, self.n_kv_heads, g, self.head_dim)
        kf = keys.float()
        vf = values.float()
        scores = torch.einsum("btkgd,bskd->bkgts", qf, kf) * (self.head_dim ** -0.5)
        scores = scores.masked_fill(~mask[:, None, None, :, :], float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        out = torch.einsum("bkgts,bskd->btkgd", probs, vf)
        return out.reshape(B, T, self.n_heads * self.head_dim).to(q.dtype)


class FeedForward(nn.Module):
    def __init__(self, args: ModelArgs):
        super().__init__()
        self.w13 = BitLinearKernel(args.dim, 2 * args.ffn_dim,
                                   seg_ends=(args.ffn_dim, 2 * args.ffn_dim) if args.segment_scales else None)
        self.w2 = BitLinearKernel(args.ffn_dim, args.dim)
        self.ffn_sub_norm = RMSNorm(args.ffn_dim, args.norm_eps)

    def forward(self, x):
        x13 = self.w13(x)
        x1, x3 = x13.chunk(2, -1)
        inner = self.ffn_sub_norm(torch.relu(x1) ** 2 * x3)  # squared-ReLU GLU, gpu/model.py:195
        return self.w2(inner)


class TransformerBlock(nn.Module):
    def __init__(self, args: ModelArgs):
        super().__init__()
        self.attention = Attention(args)
        self.feed_forward = FeedForward(args)
        self.attention_norm = RMSNorm(args.dim, args.norm_eps)
        self.ffn_norm = RMSNorm(args.dim, args.norm_eps)


class Transformer(nn.Module):
    """Decoder with an explicit KV cache [n_layers] x (k, v) of shape
    [batch, max_seq, n_kv_heads, head_dim]."""

    def __init__(self, args: ModelArgs):
        super().__init__()
        self.args = args
        self.tok_embeddings = nn.Embedding(args.vocab_size, args.dim)
        self.layers = nn.ModuleList([TransformerBlock(args) for _ in range(args.n_layers)])
        self.norm = RMSNorm(args.dim, args.norm_eps)
        self.output = nn.Linear(args.dim, args.vocab_size, bias=False)

    def make_cache(self, batch: int, max_seq: int, device, dtype=torch.bfloat16) -> List[Tuple[torch.Tensor, torch.Tensor]]:
        a = self.args
        shape = (batch, max_seq, a.n_kv_heads, a.dim // a.n_heads)
        return [(torch.zeros(shape, device=device, dtype=dtype), torch.zeros(shape, device=device, dtype=dtype))
                for _ in range(a.n_layers)]

    def fused_decode_ok(self, batch: int) -> bool:
        """One new token per sequence can take the path with the norms, the gate
        and the residual adds folded into the BitLinear calls (residual
        epilogue: up to 16 rows)."""
        a = self.args
        hd = a.dim // a.n_heads
        return hd == 128 and self.norm.weight.dtype == torch.bfloat16 and batch <= 16

    @torch.no_grad()
    def forward_decode_fused(self, tokens, positions, cache, cos, sin, workspace=None):
        """One decode step, T = 1, five kernels per layer: norm+wqkv, rope+cache+
        attention, sub-norm+wo+residual, norm+w13, gate+sub-norm+w2+residual.
        tokens / positions [B, 1].  Returns logits [B, 1, vocab] fp32."""
        h = self.decode_hidden_fused(tokens, positions, cache, cos, sin, workspace)
        return self.output(self.norm(h)).float().view(tokens.shape[0], 1, -1)

    @torch.no_grad()
    def decode_hidden_fused(self, tokens, positions, cache, cos, sin, workspace=None):
        """The decoder layers of forward_decode_fused: hidden state [B, dim] in
        front of the final norm."""
        a = self.args
        B = tokens.shape[0]
        pos = positions.reshape(B)
        if self.tok_embeddings.weight.dtype == torch.bfloat16 and a.dim % 8 == 0:
            h, rows = decode_step_begin(tokens.reshape(B), pos, self.tok_embeddings.weight, cos, sin)
        else:
            h, rows = self.tok_embeddings(tokens.reshape(B)), None
        for layer, (ck, cv) in zip(self.layers, cache):
            att, ffn = layer.attention, layer.feed_forward
            xqkv = norm_bitlinear(h, layer.attention_norm, att.wqkv)
            o = attn_decode(xqkv, ck, cv, pos, cos, sin, a.n_heads, a.n_kv_heads, workspace, rope_rows=rows)
            h = norm_bitlinear(o, att.attn_sub_norm, att.wo, residual=h)
            x13 = norm_bitlinear(h, layer.ffn_norm, ffn.w13)
            h = norm_bitlinear(x13, ffn.ffn_sub_norm, ffn.w2, glu=True, residual=h)
        return h

    @torch.no_grad()
    def prefill_hidden_fused(self, tokens, cache, cos, sin):
        """A whole prompt on an empty cache, tokens [B, T] at positions 0..T-1:
        the layer stack of decode_hidden_fused at prompt size (norms, gate and
        residual adds folded into the BitLinear calls, which run the int8 GEMM),
        rope + cache write in one kernel, causal attention over the new tokens
        in another (the reference calls xformers' rope_padded and flash attention
        here, gpu/model.py:128-155).  Returns the hidden state in front of the
        final norm, [B, T, dim]."""
        a = self.args
        B, T = tokens.shape
        pos = torch.arange(T, device=tokens.device)[None, :].expand(B, T).contiguous()
        h = self.tok_embeddings(tokens.reshape(B * T))
        for layer, (ck, cv) in zip(self.layers, cache):
            att, ffn = layer.attention, layer.feed_forward
            xqkv = norm_bitlinear(h, layer.attention_norm, att.wqkv)
            q = rope_cache_tokens(xqkv, ck, cv, pos, cos, sin, a.n_heads, a.n_kv_heads)
            o = attn_prefill(q, ck, cv, 0)
            h = norm_bitlinear(o, att.attn_sub_norm, att.wo, residual=h)
            x13 = norm_bitlinear(h, layer.ffn_norm, ffn.w13)
            h = norm_bitlinear(x13, ffn.ffn_sub_norm, ffn.w2, glu=True, residual=h)
        return h.view(B, T, a.dim)

    @torch.no_grad()
    def forward_tokens(self, tokens, positions, cache, cos, sin):
        """tokens [B, T] int64; positions [B, T] int64 (absolute position of every
        token).  Writes k/v of these tokens into the cache at their positions
        and attends to every cached position <= the token's own.  Works for
        prefill (T = prompt length) and for decode (T = 1); all shapes are
        static, so a decode step can be captured in a graph.  Returns logits
        [B, T, vocab] in fp32."""
        B, T = tokens.shape
        S = cache[0][0].shape[1]
        h = self.tok_embeddings(tokens)
        c = cos[positions][:, :, None, :]
        s = sin[positions][:, :, None, :]
        mask = torch.arange(S, device=tokens.device)[None, None, :] <= positions[:, :, None]
        bidx = torch.arange(B, device=tokens.device)[:, None].expand(B, T)
        for layer, (ck, cv) in zip(self.layers, cache):
            att = layer.attention
            q, k, v = att.split_qkv(att.wqkv(layer.attention_norm(h)))
            q = apply_rope(q, c, s)
            k = apply_rope(k, c, s)
            ck.index_put_((bidx, positions), k)
            cv.index_put_((bidx, positions), v)
            o = att.attend(q, ck, cv, mask)
            h = h + att.wo(att.attn_sub_norm(o))
            h = h + layer.feed_forward(layer.ffn_norm(h))
        return self.output(self.norm(h)).float()


def random_init_(model: Transformer, seed: int = 0) -> Transformer:
    """Random weights of the benchmark configuration: BitLinear weights ternary
    iid with P(0) = 0.4, P(+-1) = 0.3 packed in the int2 layout, one weight
    scale per sub-tensor; embedding / LM head bf16 N(0, 0.02^2), tied as the
    reference's converter ties them (gpu/convert_safetensors.py:88-89)."""
    from .pack_weight import convert_weight_int8_to_int2

    dev = model.tok_embeddings.weight.device
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    a = model.args
    hd = a.dim // a.n_heads

    def fill(mod: BitLinearKernel, parts):
        N, K = mod.out_features, mod.in_features
        u = torch.rand(N, K, generator=gen, device=dev)
        w = (u >= 0.7).to(torch.int8) - (u < 0.3).to(torch.int8)
        mod.weight.data = convert_weight_int8_to_int2(w, keep_device=True)
        sc = torch.zeros(4, dtype=torch.float32, device=dev)
        sc[: len(parts)] = 0.016 * (1.0 + 0.1 * torch.arange(len(parts), device=dev))
        mod.weight_scale.data = sc.to(torch.bfloat16)

    for layer in model.layers:
        fill(layer.attention.wqkv, (a.n_heads * hd, a.n_kv_heads * hd, a.n_kv_heads * hd))
        fill(layer.attention.wo, (a.dim,))
        fill(layer.feed_forward.w13, (a.ffn_dim, a.ffn_dim))
        fill(layer.feed_forward.w2, (a.dim,))
    emb = torch.randn(a.vocab_size, a.dim, generator=gen, device=dev) * 0.02
    model.tok_embeddings.weight.data = emb.to(model.tok_embeddings.weight.dtype)
    model.output.weight.data = model.tok_embeddings.weight.data  # tied
    return model


def top_p_sample(probs: torch.Tensor, p: float, generator: Optional[torch.Generator] = None) -> torch.Tensor:
    """Nucleus sampling, one draw per row of probs [B, V] -> int64 [B, 1]: a token
    stays in the draw while the probability mass of the tokens more likely than
    it is at most p (so the most likely token always stays, and the kept set is
    the shortest prefix of the sorted distribution whose mass exceeds p); the
    kept probabilities are renormalised by the draw itself (gpu/sample_utils.py:9-33)."""
    ranked, order = torch.sort(probs, dim=-1, descending=True)
    mass_before = torch.cumsum(ranked, dim=-1) - ranked
    kept = torch.where(mass_before > p, torch.zeros_like(ranked), ranked)
    pick = torch.multinomial(kept, num_samples=1, generator=generator)
    return torch.gather(order, -1, pick)


class Generator:
    """Greedy generation: prefill of the whole prompt in one call, then one
    graph replay per generated token (gpu/generate.py:216-288)."""

    def __init__(self, model: Transformer, batch: int, max_seq: int, use_graph: bool = True, fused: bool = True,
                 fused_head: bool = True):
        self.model = model
        self.fused = fused and model.fused_decode_ok(batch)
        a_ = model.args
        # split the cached positions of every (sequence, kv head) over up to 8 workgroups (16 for caches
        # beyond 2048 rows: measured 16.5 -> 12.3 us at 8200 rows, nothing at 642): one CU alone pulls a
        # small fraction of the memory bandwidth, and merging the splits costs about a microsecond.
        # No more workgroups than CUs (256)
        n_splits = max(1, min(16 if max_seq > 2048 else 8, 256 // max(1, batch * a_.n_kv_heads)))
        self.attn_ws = AttnWorkspace(batch, a_.n_heads, a_.n_kv_heads, n_splits, model.tok_embeddings.weight.device)
        self.batch = batch
        self.max_seq = max_seq
        dev = model.tok_embeddings.weight.device
        a = model.args
        self.cos, self.sin = rope_tables(a.dim // a.n_heads, max_seq, a.rope_theta, dev)
        self.cache = model.make_cache(batch, max_seq, dev)
        self.tok = torch.zeros(batch, 1, dtype=torch.int64, device=dev)
        self.pos = torch.zeros(batch, 1, dtype=torch.int64, device=dev)
        self.next_tok = torch.zeros(batch, dtype=torch.int64, device=dev)
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.use_graph = use_graph
        # final norm + bf16 LM head + greedy token as two launches of the library
        self.lm_head = (self.fused and fused_head and model.output.weight.dtype == torch.bfloat16 and a.dim % 64 == 0
                        and model.output.bias is None)
        self.lm_ws = LmHeadWorkspace(batch, a.vocab_size, a.dim, dev) if self.lm_head else None
        # generated tokens of a decode() call, written from inside the step so that a graph replay is the whole step
        self.history = torch.zeros(max_seq, batch, dtype=torch.int64, device=dev)
        self.step_idx = torch.zeros(1, dtype=torch.int64, device=dev)
        # captured prompt passes, one per (prompt length, logits wanted): a prompt is some three hundred launches,
        # and issued one by one from Python they cost more host time than the GPU needs for a short prompt
        # (the reference captures its prompt pass too, gpu/generate.py:102-157)
        self._pf_graphs: dict = {}
        self._rows = torch.arange(batch, device=dev)

    def _step(self):
        """One decode step including its bookkeeping: next token -> history and
        the input of the following step, position + 1."""
        if self.lm_head:
            h = self.model.decode_hidden_fused(self.tok, self.pos, self.cache, self.cos, self.sin, self.attn_ws)
            # the step's bookkeeping rides on the last kernel of the LM head
            lm_head_greedy(h, self.model.norm, self.model.output.weight, self.lm_ws, token_out=self.next_tok,
                           next_input=self.tok, positions=self.pos, history=self.history, step_idx=self.step_idx)
            return
        else:
            if self.fused:
                logits = self.model.forward_decode_fused(self.tok, self.pos, self.cache, self.cos, self.sin, self.attn_ws)
            else:
                logits = self.model.forward_tokens(self.tok, self.pos, self.cache, self.cos, self.sin)
            self.next_tok.copy_(torch.argmax(logits[:, -1, :], dim=-1))
        self.history.index_copy_(0, self.step_idx, self.next_tok.view(1, -1))
        self.step_idx.add_(1)
        self.tok.copy_(self.next_tok.view(-1, 1))
        self.pos.add_(1)

    def _capture(self):
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            self._step()  # warm-up outside the graph
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self._step()

    kMaxPrefillGraphs = 12  # captured prompt passes kept; the least recently replayed one makes room for a new one
    kPrefillBucket = 32  # prompts are padded to a multiple of this many tokens, so that lengths share captured passes

    def _bucket(self, P: int) -> int:
        b = self.kPrefillBucket
        return min(self.max_seq, (P + b - 1) // b * b)

    def _prefill_fused(self, prompt, lens, tok_out, logits):
        """The prompt through the library's kernels; only each sequence's last real token goes through the LM head."""
        h = self.model.prefill_hidden_fused(prompt, self.cache, self.cos, self.sin)
        last = h[self._rows, lens - 1].contiguous()
        return lm_head_greedy(last, self.model.norm, self.model.output.weight, self.lm_ws, token_out=tok_out, logits_out=logits)

    def _prefill_replay(self, prompt: torch.Tensor, lens: Optional[torch.Tensor], want_logits: bool):
        """prompt [B, P] (padded) through the captured pass of P's bucket: (first token [B], logits or None).
        The pass runs on the prompt padded further, with token 0, to the bucket's length; every sequence's real
        length travels in `lens` (attention is causal, so the pads change no real token's result, and the cache rows
        they write are overwritten before a decode step reads them).  The captured passes are therefore at most
        two per bucket, and beyond kMaxPrefillGraphs the least recently replayed one is dropped."""
        B, P = prompt.shape
        Pb = self._bucket(P)
        key = (Pb, want_logits)
        entry = self._pf_graphs.pop(key, None)
        if entry is None:
            while len(self._pf_graphs) >= self.kMaxPrefillGraphs:
                self._pf_graphs.pop(next(iter(self._pf_graphs)))  # dicts keep insertion order: the oldest entry
            dev = self.tok.device
            bufs = {"prompt": torch.zeros(B, Pb, dtype=torch.int64, device=dev),
                    "lens": torch.full((B,), P, dtype=torch.int64, device=dev),
                    "tok": torch.zeros(B, dtype=torch.int64, device=dev),
                    "logits": torch.empty(B, self.model.args.vocab_size, dtype=torch.float32, device=dev) if want_logits else None}
            bufs["prompt"][:, :P].copy_(prompt)
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                self._prefill_fused(bufs["prompt"], bufs["lens"], bufs["tok"], bufs["logits"])  # warm-up outside the graph
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                self._prefill_fused(bufs["prompt"], bufs["lens"], bufs["tok"], bufs["logits"])
            entry = (graph, bufs)
        self._pf_graphs[key] = entry  # (re-)inserted last: most recently used
        graph, bufs = entry
        bufs["prompt"][:, :P].copy_(prompt)
        if P < Pb:
            bufs["prompt"][:, P:].zero_()
        if lens is None:
            bufs["lens"].fill_(P)
        else:
            bufs["lens"].copy_(lens)
        graph.replay()
        return bufs["tok"].clone(), (bufs["logits"] if want_logits else None)

    @torch.no_grad()
    def prefill(self, prompt: torch.Tensor) -> torch.Tensor:
        """prompt [B, P] int64 -> first generated token [B]."""
        B, P = prompt.shape
        if self.lm_head:
            if self.use_graph and B == self.batch:
                return self._prefill_replay(prompt, None, False)[0]
            lens = torch.full((B,), P, dtype=torch.int64, device=prompt.device)
            rows = self._rows if B == self.batch else torch.arange(B, device=prompt.device)
            h = self.model.prefill_hidden_fused(prompt, self.cache, self.cos, self.sin)
            return lm_head_greedy(h[rows, lens - 1].contiguous(), self.model.norm, self.model.output.weight, self.lm_ws)
        pos = torch.arange(P, device=prompt.device)[None, :].expand(B, P).contiguous()
        logits = self.model.forward_tokens(prompt, pos, self.cache, self.cos, self.sin)
        return torch.argmax(logits[:, -1, :], dim=-1)

    def _set_positions(self, start_pos) -> None:
        if isinstance(start_pos, torch.Tensor):
            self.pos.copy_(start_pos.to(self.pos.device, torch.int64).view(-1, 1))
        else:
            self.pos.fill_(start_pos)

    @torch.no_grad()
    def decode(self, first: torch.Tensor, start_pos, steps: int, eos_id: Optional[int] = None) -> torch.Tensor:
        """Feeds `first` at position start_pos (an int, or one position per
        sequence: int64 [B], ragged prompts) and generates up to `steps` further
        tokens greedily.  With eos_id the loop ends after the first step in which
        any sequence produced that token, as the reference's loop does
        (gpu/generate.py:283-284; one device-to-host copy per step).  Returns
        [steps taken, B]."""
        if steps > self.history.shape[0]:
            raise ValueError("more steps than the generator was sized for")
        lo = int(start_pos.min()) if isinstance(start_pos, torch.Tensor) else start_pos
        hi = int(start_pos.max()) if isinstance(start_pos, torch.Tensor) else start_pos
        if isinstance(start_pos, torch.Tensor) and start_pos.numel() != self.batch:
            raise ValueError(f"decode: {start_pos.numel()} start positions for a batch of {self.batch}")
        if lo < 0 or hi + steps > self.max_seq:
            raise ValueError(f"decode: positions {lo}..{hi + steps - 1} do not fit a cache of {self.max_seq} rows")
        self.tok.copy_(first.view(-1, 1))
        self._set_positions(start_pos)
        if self.use_graph and self.graph is None:
            # capture with the real inputs in place; the captured step is re-run below
            saved_k = [ck.clone() for ck, _ in self.cache]
            saved_v = [cv.clone() for _, cv in self.cache]
            self._capture()
            for (ck, cv), sk, sv in zip(self.cache, saved_k, saved_v):
                ck.copy_(sk)
                cv.copy_(sv)
            self.tok.copy_(first.view(-1, 1))
            self._set_positions(start_pos)
        self.step_idx.zero_()
        taken = 0
        for i in range(steps):
            if self.use_graph:
                self.graph.replay()
            else:
                self._step()
            taken = i + 1
            if eos_id is not None and bool((self.next_tok == eos_id).any()):
                break
        out = self.history[:taken].clone()
        if self.fused:
            self.attn_ws.check()  # one small copy to the host per decode() call
        return out

    @torch.no_grad()
    def _prefill_ragged(self, prompts, pad_id: int, want_logits: bool):
        """Prompts of different lengths, padded on the right to the longest (attention is causal: a pad never
        reaches a real token, and the cache rows the pads leave behind are overwritten before a decode step
        reads them).  Returns (first greedy token [B], logits fp32 [B, V] or None, lengths int64 [B])."""
        dev = self.tok.device
        lens = torch.tensor([len(q) for q in prompts], dtype=torch.int64, device=dev)
        P = int(lens.max())
        prompt = torch.full((self.batch, P), pad_id, dtype=torch.int64, device=dev)
        for b, q in enumerate(prompts):
            prompt[b, : len(q)] = torch.tensor(q, dtype=torch.int64, device=dev)
        rows = self._rows
        V = self.model.args.vocab_size
        if self.lm_head:
            if self.use_graph:
                tok, logits = self._prefill_replay(prompt, lens, want_logits)
                return tok, logits, lens
            logits = torch.empty(self.batch, V, dtype=torch.float32, device=dev) if want_logits else None
            tok = self._prefill_fused(prompt, lens, None, logits)
            return tok, logits, lens
        pos = torch.arange(P, device=dev)[None, :].expand(self.batch, P).contiguous()
        logits = self.model.forward_tokens(prompt, pos, self.cache, self.cos, self.sin)[rows, lens - 1]
        return torch.argmax(logits, dim=-1), logits, lens

    @torch.no_grad()
    def generate_all(self, prompts, gen_length: int, use_sampling: bool = False, temperature: float = 0.7,
                     top_p: float = 0.95, eos_id: Optional[int] = None, pad_id: int = 1,
                     rng: Optional[torch.Generator] = None, timings: Optional[dict] = None):
        """FastGen.generate_all of the reference (gpu/generate.py:217-304) on token
        ids: `prompts` is one list of ids per sequence of the batch (lengths may
        differ; padded with pad_id, the reference's 1); the whole batch is
        prefilled in one pass, then one token per sequence and step is generated,
        greedily or -- use_sampling -- from softmax(logits / temperature) cut to
        the top_p nucleus (the reference's 0.7 / 0.95), until gen_length tokens
        are out or, with eos_id, until any sequence has produced it.  Every
        answer is cut behind its first eos_id.  Greedy steps replay the captured
        graph of the whole step; a sampled step runs the same kernels and draws
        with torch between them (`rng` makes the draws reproducible).  A dict
        passed as `timings` receives what the reference's Stats phases report
        (gpu/stats.py, gpu/generate.py:243-288): prefill_s, decode_s,
        decode_tokens (steps x sequences) and decode_tokens_per_s; it costs two
        device synchronisations."""
        if len(prompts) != self.batch:
            raise ValueError(f"generate_all: {len(prompts)} prompts for a generator of batch {self.batch}")
        if any(len(q) < 1 for q in prompts):
            raise ValueError("generate_all: empty prompt")
        longest = max(len(q) for q in prompts)
        if gen_length < 1 or longest + gen_length > self.max_seq or gen_length > self.history.shape[0]:
            raise ValueError(f"generate_all: prompt of {longest} + {gen_length} tokens does not fit a cache of {self.max_seq} rows")
        vocab = self.model.args.vocab_size
        if any(t < 0 or t >= vocab for q in prompts for t in q):
            raise ValueError("generate_all: token id outside the vocabulary")

        def draw(logits):
            probs = torch.softmax(logits / temperature, dim=-1)
            return top_p_sample(probs, top_p, rng).view(-1)

        if timings is not None:
            torch.cuda.synchronize()
            t_start = time.perf_counter()
        first, logits, lens = self._prefill_ragged(prompts, pad_id, use_sampling)
        if use_sampling:
            first = draw(logits)
        if timings is not None:
            torch.cuda.synchronize()
            t_prefill = time.perf_counter()
        out = [first.view(1, -1)]
        # (an end token that comes out of the prompt pass does not end the batch: the reference tests for it only
        # inside its decode loop, gpu/generate.py:262-284; the answers are trimmed per sequence below)
        if gen_length > 1:
            if not use_sampling:
                out.append(self.decode(first, lens, gen_length - 1, eos_id=eos_id))
            else:
                if logits is None or not self.lm_head:
                    logits = torch.empty(self.batch, vocab, dtype=torch.float32, device=self.tok.device)
                self.tok.copy_(first.view(-1, 1))
                self._set_positions(lens)
                for _ in range(gen_length - 1):
                    if self.lm_head:
                        h = self.model.decode_hidden_fused(self.tok, self.pos, self.cache, self.cos, self.sin, self.attn_ws)
                        lm_head_greedy(h, self.model.norm, self.model.output.weight, self.lm_ws, logits_out=logits)
                        step_logits = logits
                    elif self.fused:
                        step_logits = self.model.forward_decode_fused(self.tok, self.pos, self.cache, self.cos, self.sin,
                                                                      self.attn_ws)[:, -1]
                    else:
                        step_logits = self.model.forward_tokens(self.tok, self.pos, self.cache, self.cos, self.sin)[:, -1]
                    nxt = draw(step_logits)
                    out.append(nxt.view(1, -1))
                    self.tok.copy_(nxt.view(-1, 1))
                    self.pos.add_(1)
                    if eos_id is not None and bool((nxt == eos_id).any()):
                        break
                if self.fused:
                    self.attn_ws.check()
        tokens = torch.cat(out, dim=0).t().tolist()  # [B][steps]
        if timings is not None:
            torch.cuda.synchronize()
            t_end = time.perf_counter()
            steps = len(tokens[0]) - 1
            timings.update(prefill_s=t_prefill - t_start, decode_s=t_end - t_prefill, decode_tokens=steps * self.batch,
                           decode_tokens_per_s=(steps * self.batch / (t_end - t_prefill)) if steps else 0.0)
        answers = []
        for ans in tokens:
            if eos_id is not None and eos_id in ans:
                ans = ans[: ans.index(eos_id) + 1]
            answers.append(ans)
        return answers
