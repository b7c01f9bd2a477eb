"""Decoder (the caller of the hot path) on a small configuration: the library
BitLinear inside the full layer stack against a torch emulation of the same
arithmetic, prefill/decode consistency, and the graph-replayed decode loop."""
import numpy as np
import pytest
import torch

from bitnet_amd import _lib, decoder, pack_weight
from bitnet_amd.bitlinear import BitLinearKernel
from tests.gpu_util import host_bits
from oracle import bitlinear_oracle as o

pytestmark = pytest.mark.gpu

SMALL = decoder.ModelArgs(dim=256, n_layers=3, n_heads=4, n_kv_heads=2, vocab_size=512, ffn_dim=512)


class RefBitLinear(torch.nn.Module):
    """gpu/model.py:68-75 + bitnet_kernels.h:79-82 in plain torch: compiled-mode
    quantizer (reciprocal, multiply, bf16 scale, exact fp32 product), exact
    integer product in float64, fp32 divide / multiply / RNE epilogue with the
    equal-slot scale rule."""

    def __init__(self, mod: BitLinearKernel, ws_num: int):
        super().__init__()
        self.w = pack_weight.convert_weight_int2_to_int8(mod.weight.data, mod.out_features, mod.in_features).double()
        self.ws = mod.weight_scale.data.float()
        self.slot = torch.arange(mod.out_features, device=self.w.device) // (mod.out_features // ws_num)

    def forward(self, x):
        xf = x.float()
        amax = xf.abs().amax(dim=-1, keepdim=True).clamp(min=1e-5)
        s = ((1.0 / amax) * 127.0).to(torch.bfloat16).float()
        q = (xf * s).round().clamp(-128, 127)
        acc = (q.double() @ self.w.T).float()
        return (acc / s * self.ws[self.slot]).to(torch.bfloat16)


def _build(args, seed=0):
    torch.manual_seed(seed)
    with torch.device("cuda"):
        prev = torch.get_default_dtype()
        torch.set_default_dtype(torch.bfloat16)
        try:
            model = decoder.Transformer(args)
        finally:
            torch.set_default_dtype(prev)
    return decoder.random_init_(model, seed)


def _reference_copy(model):
    import copy

    ref = copy.deepcopy(model)
    for lr in ref.layers:
        lr.attention.wqkv = RefBitLinear(lr.attention.wqkv, 1)  # shapes outside the reference's table: one slot
        lr.attention.wo = RefBitLinear(lr.attention.wo, 1)
        lr.feed_forward.w13 = RefBitLinear(lr.feed_forward.w13, 1)
        lr.feed_forward.w2 = RefBitLinear(lr.feed_forward.w2, 1)
    return ref


def test_state_dict_names_match_the_reference_checkpoint_layout():
    model = _build(SMALL)
    keys = set(model.state_dict().keys())
    for k in ["tok_embeddings.weight", "norm.weight", "output.weight", "layers.0.attention.wqkv.weight",
              "layers.0.attention.wqkv.weight_scale", "layers.0.attention.wo.weight", "layers.0.attention.attn_sub_norm.weight",
              "layers.0.feed_forward.w13.weight", "layers.0.feed_forward.w2.weight_scale",
              "layers.0.feed_forward.ffn_sub_norm.weight", "layers.0.attention_norm.weight", "layers.0.ffn_norm.weight"]:
        assert k in keys, k
    assert model.layers[0].attention.wqkv.weight.shape == (512, 64) and model.layers[0].attention.wqkv.weight.dtype == torch.int8


def test_logits_equal_torch_emulation_prefill_and_decode():
    model = _build(SMALL, seed=1)
    ref = _reference_copy(model)
    B, P, S = 2, 24, 40
    dev = torch.device("cuda")
    cos, sin = decoder.rope_tables(SMALL.dim // SMALL.n_heads, S, SMALL.rope_theta, dev)
    g = torch.Generator(device="cuda").manual_seed(5)
    prompt = torch.randint(0, SMALL.vocab_size, (B, P), generator=g, device=dev)
    pos = torch.arange(P, device=dev)[None].expand(B, P).contiguous()
    c1, c2 = model.make_cache(B, S, dev), ref.make_cache(B, S, dev)
    l1 = model.forward_tokens(prompt, pos, c1, cos, sin)   # M = 48: quantizer kernel + MFMA GEMM
    l2 = ref.forward_tokens(prompt, pos, c2, cos, sin)
    assert torch.equal(l1, l2)
    tok = torch.argmax(l1[:, -1], dim=-1).view(B, 1)
    p1 = torch.full((B, 1), P, device=dev)
    d1 = model.forward_tokens(tok, p1, c1, cos, sin)        # M = 2: fused one-kernel forward
    d2 = ref.forward_tokens(tok, p1, c2, cos, sin)
    assert torch.equal(d1, d2)
    for (k1, v1), (k2, v2) in zip(c1, c2):
        assert torch.equal(k1, k2) and torch.equal(v1, v2)


def test_decode_step_equals_prefill_of_the_longer_prompt():
    model = _build(SMALL, seed=2)
    B, P, S = 1, 17, 32
    dev = torch.device("cuda")
    cos, sin = decoder.rope_tables(SMALL.dim // SMALL.n_heads, S, SMALL.rope_theta, dev)
    g = torch.Generator(device="cuda").manual_seed(6)
    ids = torch.randint(0, SMALL.vocab_size, (B, P + 1), generator=g, device=dev)
    pos = torch.arange(P + 1, device=dev)[None]
    full = model.forward_tokens(ids, pos, model.make_cache(B, S, dev), cos, sin)[:, -1]
    cache = model.make_cache(B, S, dev)
    model.forward_tokens(ids[:, :P], pos[:, :P], cache, cos, sin)
    step = model.forward_tokens(ids[:, P:], pos[:, P:], cache, cos, sin)[:, -1]
    # every op is per token except attention, whose cache holds the same keys/values
    assert torch.equal(full, step)


def test_graph_decode_loop_equals_eager_loop():
    model = _build(SMALL, seed=3)
    B, P, G = 2, 16, 12
    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(7)
    prompt = torch.randint(0, SMALL.vocab_size, (B, P), generator=g, device=dev)
    outs = []
    for use_graph in (False, True):
        gen = decoder.Generator(model, B, P + G + 1, use_graph=use_graph)
        first = gen.prefill(prompt)
        toks = gen.decode(first, P, G)
        torch.cuda.synchronize()
        outs.append(torch.cat([first[None], toks]).cpu())
    assert torch.equal(outs[0], outs[1])
    assert outs[0].shape == (G + 1, B)


BIG_HEADS = decoder.ModelArgs(dim=512, n_layers=2, n_heads=4, n_kv_heads=1, vocab_size=256, ffn_dim=768)  # head_dim 128


def _ulp(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    def mono(t):
        v = t.view(torch.int16).to(torch.int32)
        return torch.where(v < 0, -(v & 0x7FFF), v)
    return (mono(a) - mono(b)).abs()


@pytest.mark.parametrize("n_splits", [1, 3, 8])
@pytest.mark.parametrize("B,S,nh,nkv", [(1, 641, 20, 5), (8, 200, 20, 5), (2, 64, 4, 1), (3, 1500, 8, 8), (2, 33, 16, 2)])
def test_attention_decode_kernel_against_torch_fp32(B, S, nh, nkv, n_splits):
    """A floating-point kernel: compared with the fp32 torch restatement (rope,
    cache write, softmax(QK^T/sqrt(d))V).  Its probabilities are rounded to
    bf16 for the matrix pipe and its fp32 sums run in another order: 3 bf16 ulp
    or 4e-3 absolute on the bf16 outputs."""
    hd = 128
    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(B * 1000 + S)
    args = decoder.ModelArgs(dim=nh * hd, n_heads=nh, n_kv_heads=nkv, n_layers=1, vocab_size=16, ffn_dim=256)
    att = decoder.Attention.__new__(decoder.Attention)
    torch.nn.Module.__init__(att)
    att.head_dim, att.n_heads, att.n_kv_heads = hd, nh, nkv
    xqkv = torch.randn(B, (nh + 2 * nkv) * hd, generator=g, device=dev).to(torch.bfloat16)
    ck = torch.randn(B, S, nkv, hd, generator=g, device=dev).to(torch.bfloat16)
    cv = torch.randn(B, S, nkv, hd, generator=g, device=dev).to(torch.bfloat16)
    pos = torch.randint(0, S, (B,), generator=g, device=dev)
    pos[0] = S - 1
    if B > 1:
        pos[1] = 0
    cos, sin = decoder.rope_tables(hd, S, 500000.0, dev)
    # reference
    q, k, v = att.split_qkv(xqkv[:, None, :])
    c, s_ = cos[pos][:, None, None, :], sin[pos][:, None, None, :]
    q, k = decoder.apply_rope(q, c, s_), decoder.apply_rope(k, c, s_)
    rk, rv = ck.clone(), cv.clone()
    bidx = torch.arange(B, device=dev)
    rk[bidx, pos] = k[:, 0]
    rv[bidx, pos] = v[:, 0]
    mask = torch.arange(S, device=dev)[None, None, :] <= pos[:, None, None]
    want = att.attend(q, rk, rv, mask)[:, 0]
    ws = decoder.AttnWorkspace(B, nh, nkv, n_splits, dev) if n_splits > 1 else None
    got = decoder.attn_decode(xqkv, ck, cv, pos, cos, sin, nh, nkv, ws)
    torch.cuda.synchronize()
    assert torch.equal(ck, rk) and torch.equal(cv, rv)  # cache rows written exactly
    if ws is not None:
        again = decoder.attn_decode(xqkv, ck, cv, pos, cos, sin, nh, nkv, ws)  # same cache row rewritten
        assert torch.equal(again, got)
    # the same call with the positions' cos | sin rows handed over: identical bits
    emb = torch.randn(16, 64, generator=g, device=dev).to(torch.bfloat16)
    toks = torch.randint(0, 16, (B,), generator=g, device=dev)
    h0, rows = decoder.decode_step_begin(toks, pos, emb, cos, sin)
    assert torch.equal(h0, emb[toks]) and torch.equal(rows, torch.cat([cos[pos], sin[pos]], dim=1))
    ck2, cv2 = ck.clone(), cv.clone()
    with_rows = decoder.attn_decode(xqkv, ck2, cv2, pos, cos, sin, nh, nkv, ws, rope_rows=rows)
    torch.cuda.synchronize()
    assert torch.equal(with_rows, got) and torch.equal(ck2, rk) and torch.equal(cv2, rv)
    ulps, tol = 3, 4e-3
    bad = (_ulp(got, want) > ulps) & ((got.float() - want.float()).abs() > tol)
    assert not bad.any(), f"{int(bad.sum())} of {bad.numel()} outside tolerance"


@pytest.mark.parametrize("n_splits", [5, 16])
@pytest.mark.parametrize("p", [0, 31, 32, 511, 600, 2047, 4099])
def test_attention_decode_long_cache_any_position(p, n_splits):
    """Cache capacity far beyond the position (4100 rows, up to 16 splits, eight
    waves per workgroup): the rows are dealt to splits and waves in blocks of
    32, so positions at block edges, inside the first round and in later rounds
    are covered.  Same comparison and tolerance as above (matrix-pipe kernel)."""
    B, S, nh, nkv, hd = 2, 4100, 8, 2, 128
    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(77 + p)
    att = decoder.Attention.__new__(decoder.Attention)
    torch.nn.Module.__init__(att)
    att.head_dim, att.n_heads, att.n_kv_heads = hd, nh, nkv
    xqkv = torch.randn(B, (nh + 2 * nkv) * hd, generator=g, device=dev).to(torch.bfloat16)
    ck = torch.randn(B, S, nkv, hd, generator=g, device=dev).to(torch.bfloat16)
    cv = torch.randn(B, S, nkv, hd, generator=g, device=dev).to(torch.bfloat16)
    pos = torch.tensor([p, max(0, p - 17)], device=dev)
    cos, sin = decoder.rope_tables(hd, S, 500000.0, dev)
    q, k, v = att.split_qkv(xqkv[:, None, :])
    c, s_ = cos[pos][:, None, None, :], sin[pos][:, None, None, :]
    q, k = decoder.apply_rope(q, c, s_), decoder.apply_rope(k, c, s_)
    rk, rv = ck.clone(), cv.clone()
    bidx = torch.arange(B, device=dev)
    rk[bidx, pos] = k[:, 0]
    rv[bidx, pos] = v[:, 0]
    mask = torch.arange(S, device=dev)[None, None, :] <= pos[:, None, None]
    want = att.attend(q, rk, rv, mask)[:, 0]
    ws = decoder.AttnWorkspace(B, nh, nkv, n_splits, dev)
    got = decoder.attn_decode(xqkv, ck, cv, pos, cos, sin, nh, nkv, ws)
    again = decoder.attn_decode(xqkv, ck, cv, pos, cos, sin, nh, nkv, ws)
    torch.cuda.synchronize()
    assert torch.equal(ck, rk) and torch.equal(cv, rv) and torch.equal(again, got)
    bad = (_ulp(got, want) > 3) & ((got.float() - want.float()).abs() > 4e-3)
    assert not bad.any(), f"{int(bad.sum())} of {bad.numel()} outside tolerance"


@pytest.mark.parametrize("n_splits", [1, 8])
def test_attention_decode_ignores_rows_behind_the_position(n_splits):
    """Cache rows behind a sequence's position may never have been written:
    with NaNs there the output has the bits it has with finite values there."""
    B, S, nh, nkv, hd = 3, 300, 8, 2, 128
    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(4242)
    xqkv = torch.randn(B, (nh + 2 * nkv) * hd, generator=g, device=dev).to(torch.bfloat16)
    ck = torch.randn(B, S, nkv, hd, generator=g, device=dev).to(torch.bfloat16)
    cv = torch.randn(B, S, nkv, hd, generator=g, device=dev).to(torch.bfloat16)
    pos = torch.tensor([0, 37, 255], device=dev)
    cos, sin = decoder.rope_tables(hd, S, 500000.0, dev)
    ws = decoder.AttnWorkspace(B, nh, nkv, n_splits, dev) if n_splits > 1 else None
    want = decoder.attn_decode(xqkv, ck.clone(), cv.clone(), pos, cos, sin, nh, nkv, ws)
    behind = torch.arange(S, device=dev)[None, :] > pos[:, None]
    ck[behind] = float("nan")
    cv[behind] = float("nan")
    got = decoder.attn_decode(xqkv, ck, cv, pos, cos, sin, nh, nkv, ws)
    torch.cuda.synchronize()
    assert not torch.isnan(got.float()).any()
    assert torch.equal(got, want)
    assert torch.isnan(ck[behind].float()).all() and torch.isnan(cv[behind].float()).all()


def test_fused_decode_path_against_unfused():
    """Five-kernels-per-layer decode step vs the torch-glue step on a small model
    with 128-wide heads: every sub-step on identical inputs (bit-level bounds, see
    _decode_step_substeps_against_glue), and over a short generation the same
    greedy tokens most of the time (each path's quantizers amplify the other's
    rounding differences, so the token streams may part at a near tie)."""
    model = _build(BIG_HEADS, seed=4)
    assert model.fused_decode_ok(2)
    B, P, G = 2, 20, 8
    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(9)
    prompt = torch.randint(0, BIG_HEADS.vocab_size, (B, P), generator=g, device=dev)
    outs = []
    for fused in (False, True):
        gen = decoder.Generator(model, B, P + G + 1, use_graph=fused, fused=fused)
        first = gen.prefill(prompt)
        outs.append(torch.cat([first[None], gen.decode(first, P, G)]).cpu())
    torch.cuda.synchronize()
    assert (outs[0] == outs[1]).float().mean() > 0.8
    gen = decoder.Generator(model, B, P + G + 1)
    first = gen.prefill(prompt)
    h, hc, worst = _decode_step_substeps_against_glue(model, gen, first.view(B, 1), P)
    cosine = torch.nn.functional.cosine_similarity(model.output(model.norm(h)).float(), model.output(model.norm(hc)).float(), dim=-1)
    assert float(cosine.min()) > 0.99, (float(cosine.min()), worst)


@pytest.mark.parametrize("which", [0, 1])
@pytest.mark.parametrize("B,V,K", [(1, 128256, 2560), (8, 128256, 2560), (3, 1000, 256), (16, 4111, 512), (2, 48, 64),
                                   (2, 4111, 512), (4, 77, 1024), (5, 32000, 2048)])
def test_lm_head_greedy_kernel(B, V, K, which):
    """Final norm + bf16 LM head + greedy token: the normalised rows bit-exact
    against the oracle's RMSNorm, the logits within one bf16 ulp (or 1e-3 of
    the largest logit, where sums cancel) of an fp32 torch evaluation (fp32
    sums in another order), the token equal to the first maximum of the
    kernel's own logits."""
    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(B * 7 + V)
    h = (torch.randn(B, K, generator=g, device=dev) * 3).to(torch.bfloat16)
    emb = (torch.randn(V, K, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    norm = decoder.RMSNorm(K, 1e-5).to(dev)
    norm.weight.data = (1 + 0.1 * torch.randn(K, generator=g, device=dev)).to(torch.bfloat16)
    ws = decoder.LmHeadWorkspace(B, V, K, dev)
    logits = torch.full((B, V), float("nan"), dtype=torch.float32, device=dev)
    lib = _lib.load_library()
    assert lib.bitnet_lm_head_set_kernel(which) == 0  # 0: built-in choice (streaming kernel where it applies), 1: MFMA kernel
    try:
        tok = decoder.lm_head_greedy(h, norm, emb, ws, logits_out=logits)
        torch.cuda.synchronize()
    finally:
        lib.bitnet_lm_head_set_kernel(0)
    want_y = o.rmsnorm_bf16(host_bits(h), host_bits(norm.weight.data), 1e-5)
    assert np.array_equal(host_bits(ws.y), want_y)
    ref = (ws.y.float() @ emb.float().T).to(torch.bfloat16)
    got = logits.to(torch.bfloat16)
    assert torch.equal(got.float(), logits)  # the kernel's logits are bf16 values
    bad = (_ulp(got, ref) > 1) & ((got.float() - ref.float()).abs() > 1e-3 * float(ref.float().abs().max()))
    assert not bad.any(), f"{int(bad.sum())} of {bad.numel()} logits outside tolerance"
    assert torch.equal(tok, torch.argmax(logits, dim=-1))
    # without the logits buffer, and a second call on the same scratch
    tok2 = decoder.lm_head_greedy(h, norm, emb, ws)
    assert torch.equal(tok2, tok)


def test_generator_with_and_without_the_lm_head_kernel_agree():
    args = decoder.ModelArgs(dim=256, n_layers=2, n_heads=2, n_kv_heads=1, vocab_size=512, ffn_dim=512)
    model = _build(args, seed=3)
    prompt = torch.randint(0, args.vocab_size, (2, 9), generator=torch.Generator().manual_seed(5)).cuda()
    outs = []
    for fused_head in (True, False):
        gen = decoder.Generator(model, 2, 40, use_graph=True, fused_head=fused_head)
        assert gen.lm_head == fused_head
        first = gen.prefill(prompt)
        outs.append(gen.decode(first, 9, 12).cpu())
    # greedy tokens can only differ where two logits tie within fp32 summation order; with random weights they do not
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("B,T,S,nh,nkv,start", [(1, 512, 640, 20, 5, 0), (3, 37, 64, 4, 1, 5), (2, 1, 16, 8, 8, 15)])
def test_rope_cache_tokens_kernel_equals_torch(B, T, S, nh, nkv, start):
    """Rope + cache write for a block of tokens: the rotated q and the cache
    rows equal the torch restatement bit for bit (fp32 products, one fp32
    add, one rounding to bf16), other cache rows untouched."""
    hd = 128
    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(B * 100 + T)
    xqkv = torch.randn(B * T, (nh + 2 * nkv) * hd, generator=g, device=dev).to(torch.bfloat16)
    ck = torch.randn(B, S, nkv, hd, generator=g, device=dev).to(torch.bfloat16)
    cv = torch.randn(B, S, nkv, hd, generator=g, device=dev).to(torch.bfloat16)
    pos = (start + torch.arange(T, device=dev))[None, :].expand(B, T).contiguous()
    cos, sin = decoder.rope_tables(hd, S, 500000.0, dev)
    att = decoder.Attention.__new__(decoder.Attention)
    torch.nn.Module.__init__(att)
    att.head_dim, att.n_heads, att.n_kv_heads = hd, nh, nkv
    q, k, v = att.split_qkv(xqkv.view(B, T, -1))
    c, s_ = cos[pos][:, :, None, :], sin[pos][:, :, None, :]
    want_q, want_k = decoder.apply_rope(q, c, s_), decoder.apply_rope(k, c, s_)
    rk, rv = ck.clone(), cv.clone()
    rk[:, start:start + T] = want_k
    rv[:, start:start + T] = v
    got_q = decoder.rope_cache_tokens(xqkv, ck, cv, pos, cos, sin, nh, nkv)
    torch.cuda.synchronize()
    assert torch.equal(got_q, want_q)
    assert torch.equal(ck, rk) and torch.equal(cv, rv)


def test_prompt_through_the_library_kernels_against_the_torch_glue():
    """Generator.prefill with the prompt-sized layer stack (norm / gate /
    residual folded into the BitLinear calls, rope + cache kernel, the prompt
    attention kernel) against forward_tokens (every op in torch around the same
    BitLinear kernels, fp32 attention): the first layer's cache rows and the
    last token's logits within bf16 noise (the norm's and the attention's sums
    run in another order and precision), and each path's first token equal to
    the argmax of its own logits."""
    model = _build(BIG_HEADS, seed=11)
    B, P, S = 2, 70, 96
    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(12)
    prompt = torch.randint(0, BIG_HEADS.vocab_size, (B, P), generator=g, device=dev)
    cos, sin = decoder.rope_tables(128, S, BIG_HEADS.rope_theta, dev)
    c1, c2 = model.make_cache(B, S, dev), model.make_cache(B, S, dev)
    h1 = model.prefill_hidden_fused(prompt, c1, cos, sin)
    pos = torch.arange(P, device=dev)[None].expand(B, P).contiguous()
    logits2 = model.forward_tokens(prompt, pos, c2, cos, sin)
    torch.cuda.synchronize()
    for a_, b_ in zip(c1[0], c2[0]):  # the two RMSNorm evaluations differ in the last bf16 bit of a few elements
        assert torch.allclose(a_.float(), b_.float(), rtol=2e-2, atol=2e-2)
        assert torch.equal(a_[:, P:], b_[:, P:])  # rows behind the prompt untouched
    logits1 = model.output(model.norm(h1[:, -1])).float()
    assert torch.allclose(logits1, logits2[:, -1], rtol=5e-2, atol=5e-2)
    gen = decoder.Generator(model, B, S)
    assert gen.lm_head
    first = gen.prefill(prompt)
    assert torch.equal(first, torch.argmax(logits1, dim=-1))
    gen2 = decoder.Generator(model, B, S, fused_head=False)
    assert torch.equal(gen2.prefill(prompt), torch.argmax(logits2[:, -1], dim=-1))


@pytest.mark.parametrize("B,T,S,nh,nkv,start", [(1, 512, 640, 20, 5, 0), (2, 70, 96, 4, 1, 0), (3, 33, 80, 8, 8, 40),
                                               (1, 1, 16, 16, 2, 9), (2, 200, 256, 8, 4, 17), (1, 16, 16, 2, 2, 0)])
def test_attention_prefill_kernel_against_torch_fp32(B, T, S, nh, nkv, start):
    """Floating-point kernel: compared with the fp32 torch restatement
    softmax(QK^T/sqrt(d))V over cache rows 0..start+t.  The kernel rounds the
    probabilities to bf16 for the matrix pipe (relative error 2^-9 each), so
    the tolerance is 3 bf16 ulp or 4e-3 absolute on the bf16 outputs.  Cache
    rows behind the last position hold NaNs: they must not be touched."""
    hd = 128
    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(B * 1000 + T + start)
    q = torch.randn(B, T, nh, hd, generator=g, device=dev).to(torch.bfloat16)
    ck = torch.randn(B, S, nkv, hd, generator=g, device=dev).to(torch.bfloat16)
    cv = torch.randn(B, S, nkv, hd, generator=g, device=dev).to(torch.bfloat16)
    ck[:, start + T:] = float("nan")
    cv[:, start + T:] = float("nan")
    att = decoder.Attention.__new__(decoder.Attention)
    torch.nn.Module.__init__(att)
    att.head_dim, att.n_heads, att.n_kv_heads = hd, nh, nkv
    pos = start + torch.arange(T, device=dev)
    mask = (torch.arange(start + T, device=dev)[None, None, :] <= pos[None, :, None]).expand(B, T, start + T)
    want = att.attend(q, ck[:, :start + T], cv[:, :start + T], mask).reshape(B * T, nh * hd)
    got = decoder.attn_prefill(q, ck, cv, start)
    torch.cuda.synchronize()
    assert not torch.isnan(got.float()).any()
    bad = (_ulp(got, want) > 3) & ((got.float() - want.float()).abs() > 4e-3)
    assert not bad.any(), f"{int(bad.sum())} of {bad.numel()} outside tolerance, max abs {float((got.float() - want.float()).abs().max())}"


def test_attention_merge_that_gives_up_is_reported():
    """The bounded poll of the merging workgroup, forced to run out from the
    host (a bound of zero polls: every kernel still runs to its end): the
    affected output rows are NaN, the workspace's error word is set and stays
    set, AttnWorkspace.check() raises; with the built-in bound restored and a
    fresh workspace the same call is healthy again."""
    B, S, nh, nkv, hd, n_splits = 2, 400, 8, 2, 128, 4
    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(99)
    xqkv = torch.randn(B, (nh + 2 * nkv) * hd, generator=g, device=dev).to(torch.bfloat16)
    ck = torch.randn(B, S, nkv, hd, generator=g, device=dev).to(torch.bfloat16)
    cv = torch.randn(B, S, nkv, hd, generator=g, device=dev).to(torch.bfloat16)
    pos = torch.tensor([399, 5], device=dev)  # sequence 1 sees one block of rows only: a single active split, nothing to merge
    cos, sin = decoder.rope_tables(hd, S, 500000.0, dev)
    lib = _lib.load_library()
    ws = decoder.AttnWorkspace(B, nh, nkv, n_splits, dev)
    assert ws.error() == 0
    good = decoder.attn_decode(xqkv, ck.clone(), cv.clone(), pos, cos, sin, nh, nkv, ws)
    torch.cuda.synchronize()
    assert ws.error() == 0 and not torch.isnan(good.float()).any()
    try:
        assert lib.bitnet_attn_decode_set_spin_limit(0) == 0
        bad = decoder.attn_decode(xqkv, ck.clone(), cv.clone(), pos, cos, sin, nh, nkv, ws)
        torch.cuda.synchronize()
    finally:
        lib.bitnet_attn_decode_set_spin_limit(-1)
    assert torch.isnan(bad[0].float()).all()           # every head of the sequence whose splits had to be merged
    assert torch.equal(bad[1], good[1])                # the single-split sequence is not affected
    assert ws.error() == 1
    again = decoder.attn_decode(xqkv, ck.clone(), cv.clone(), pos, cos, sin, nh, nkv, ws)
    torch.cuda.synchronize()
    assert torch.equal(again, good) and ws.error() == 1  # results recover; the word stays until someone looks
    with pytest.raises(_lib.BitLinearLibraryError):
        ws.check()
    assert ws.error() == 0                              # reported once: check() put the workspace back to its fresh state
    ws.check()
    once_more = decoder.attn_decode(xqkv, ck.clone(), cv.clone(), pos, cos, sin, nh, nkv, ws)
    torch.cuda.synchronize()
    assert torch.equal(once_more, good) and ws.error() == 0
    ws2 = decoder.AttnWorkspace(B, nh, nkv, n_splits, dev)
    fresh = decoder.attn_decode(xqkv, ck.clone(), cv.clone(), pos, cos, sin, nh, nkv, ws2)
    assert torch.equal(fresh, good) and ws2.error() == 0


def test_attention_decode_clamps_positions_outside_the_cache():
    """A position outside [0, S) must not take any access outside the buffers:
    the kernel clamps it.  Checked on outputs and buffers only: a position of
    S + 1000 (or 2^40) behaves exactly like S - 1, a negative one like 0, and
    guard rows allocated around the cache keep their bytes."""
    B, S, nh, nkv, hd = 3, 96, 8, 2, 128
    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(31337)
    xqkv = torch.randn(B, (nh + 2 * nkv) * hd, generator=g, device=dev).to(torch.bfloat16)
    guard = 8
    big_k = torch.randn(B + 2, S + 2 * guard, nkv, hd, generator=g, device=dev).to(torch.bfloat16)
    big_v = torch.randn(B + 2, S + 2 * guard, nkv, hd, generator=g, device=dev).to(torch.bfloat16)

    def caches():
        # a contiguous [B, S, ...] cache cut out of the middle of a larger allocation
        k = big_k.clone()
        v = big_v.clone()
        flat_k = k.view(-1)[(S + 2 * guard) * nkv * hd:][: B * S * nkv * hd].view(B, S, nkv, hd)
        flat_v = v.view(-1)[(S + 2 * guard) * nkv * hd:][: B * S * nkv * hd].view(B, S, nkv, hd)
        return k, v, flat_k, flat_v

    cos, sin = decoder.rope_tables(hd, S, 500000.0, dev)
    outs = []
    for pos_list in ([S + 1000, -7, 1 << 40], [S - 1, 0, S - 1]):
        k, v, ck, cv = caches()
        pos = torch.tensor(pos_list, device=dev, dtype=torch.int64)
        ws = decoder.AttnWorkspace(B, nh, nkv, 4, dev)
        out = decoder.attn_decode(xqkv, ck, cv, pos, cos, sin, nh, nkv, ws)
        torch.cuda.synchronize()
        outs.append((out, k, v))
    (o_bad, k_bad, v_bad), (o_ok, k_ok, v_ok) = outs
    assert not torch.isnan(o_bad.float()).any()
    assert torch.equal(o_bad, o_ok)
    assert torch.equal(k_bad, k_ok) and torch.equal(v_bad, v_ok)  # same rows written, nothing outside
    # everything outside the [B, S] window is untouched
    n_front = (S + 2 * guard) * nkv * hd
    n_win = B * S * nkv * hd
    for got, src in ((k_bad, big_k), (v_bad, big_v)):
        assert torch.equal(got.view(-1)[:n_front], src.view(-1)[:n_front])
        assert torch.equal(got.view(-1)[n_front + n_win:], src.view(-1)[n_front + n_win:])


def test_host_checks_refuse_mismatched_buffers_before_any_launch():
    dev = torch.device("cuda")
    B, S, nh, nkv, hd = 2, 32, 4, 1, 128
    xqkv = torch.zeros(B, (nh + 2 * nkv) * hd, dtype=torch.bfloat16, device=dev)
    ck = torch.zeros(B, S, nkv, hd, dtype=torch.bfloat16, device=dev)
    cv = torch.zeros_like(ck)
    pos = torch.zeros(B, dtype=torch.int64, device=dev)
    cos, sin = decoder.rope_tables(hd, S, 500000.0, dev)
    ws3 = decoder.AttnWorkspace(3, nh, nkv, 2, dev)
    with pytest.raises(ValueError):
        decoder.attn_decode(xqkv, ck, cv, pos, cos, sin, nh, nkv, ws3)          # workspace of another batch
    with pytest.raises(ValueError):
        decoder.attn_decode(xqkv, ck[:1], cv[:1], pos, cos, sin, nh, nkv)       # cache of another batch
    with pytest.raises(ValueError):
        decoder.attn_decode(xqkv[:, :-128].contiguous(), ck, cv, pos, cos, sin, nh, nkv)
    mod = BitLinearKernel(256, 64).cuda()
    with pytest.raises(ValueError):
        mod(torch.zeros(2, 192, dtype=torch.bfloat16, device=dev))               # short last dimension
    with pytest.raises(TypeError):
        mod(torch.zeros(2, 256, dtype=torch.float16, device=dev))
    model = _build(SMALL, seed=5)
    gen = decoder.Generator(model, 1, 16)
    first = torch.zeros(1, dtype=torch.int64, device=dev)
    with pytest.raises(ValueError):
        gen.decode(first, 10, 8)                                                 # positions 10..17 in a cache of 16 rows


# ---------------------------------------------------------------------------
# The end-to-end workload at its real size: 30 layers, dim 2560, ffn 6912, 20 / 5 heads, vocabulary
# 128256 (gpu/model.py:39-49), a 512-token seeded prompt, greedy decode (gpu/generate.py:264-288)
# ---------------------------------------------------------------------------
@pytest.fixture(scope="module")
def model_2b():
    model = _build(decoder.ModelArgs(), seed=0)
    yield model
    del model
    torch.cuda.empty_cache()


def _rel_l2(a, b):
    return float((a.float() - b.float()).norm() / b.float().norm())


@pytest.mark.parametrize("B", [1, 8])
def test_full_size_decoder_graph_loop_equals_eager_loop(model_2b, B):
    """512-token prompt, then 128 generated tokens as the end-to-end workload names them (the first from the
    prompt pass, 127 greedy steps): the graph-replayed loop and the eager loop run the same kernels on the same
    data, so the tokens must be identical; so must a second generation from the same prompt."""
    P, G = 512, 127
    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(1234 + B)
    prompt = torch.randint(0, model_2b.args.vocab_size, (B, P), generator=g, device=dev)
    outs = []
    for use_graph in (False, True, True):
        gen = decoder.Generator(model_2b, B, P + G + 1, use_graph=use_graph)
        assert gen.fused and gen.lm_head
        first = gen.prefill(prompt)
        toks = gen.decode(first, P, G)
        torch.cuda.synchronize()
        outs.append(torch.cat([first[None], toks]).cpu())
        del gen
    assert outs[0].shape == (G + 1, B)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[1], outs[2])
    assert int(outs[0].min()) >= 0 and int(outs[0].max()) < model_2b.args.vocab_size
    assert torch.unique(outs[0]).numel() > 4  # not a constant stream


def _decode_step_substeps_against_glue(model, gen, tok, P):
    """One decode step at position P along the fused path (five library kernels
    per layer).  Every sub-step of every layer is also evaluated the torch-glue
    way (torch RMSNorm / gate / residual around the same BitLinear kernels; torch
    rope + fp32 attention) ON THE FUSED PATH'S INPUT of that sub-step, so that
    differences cannot travel.  Returns the fused hidden state, the glue path's
    own chained hidden state, and the worst distances seen.

    What may differ within a sub-step:
      * norm -> quantizer -> product -> epilogue [-> residual]: the same
        arithmetic on both sides except the RMSNorm's sum of squares (fp64 in the
        library, fp32 in torch's order).  The fp32 mean then differs by a few
        units in the last place, which flips the bf16 rounding of a normalised
        element with probability of about 1e-4 per element; a flipped element
        moves one int8 code by one step, an accumulator by 1 in about 1500, and
        with it roughly every sixth output of that row by one bf16 ulp.
        Asserted: relative L2 distance of the sub-step's output at most 2^-8
        (one or two flipped elements stay below half of that).
      * attention: the library kernel rounds probabilities to bf16 for the matrix
        pipe (2^-9 relative each); the glue keeps fp32.  Asserted: the bound of
        the kernel's own test, 3 bf16 ulp or 4e-3 absolute per element.
    Over a whole layer the attention's 1e-3 relative difference does NOT stay
    that small: each absmax quantizer behind it rounds to a grid of 1/127 of the
    row maximum (about 3 % of a typical element), so a perturbation far below the
    grid step flips the rounding of a share of the elements by a whole step, and
    the relu^2 gate doubles relative changes.  Measured at the 2B size: 1-3 % per
    layer.  That is the conditioning of int8 activation quantization (the same
    would separate the reference's own fp prefill from its int8 decode), not a
    property of either implementation, which is why the sub-steps are compared on
    identical inputs."""
    a = model.args
    B = tok.shape[0]
    dev = tok.device
    pos = torch.full((B, 1), P, device=dev, dtype=torch.int64)
    cos, sin = gen.cos, gen.sin
    c = cos[pos][:, :, None, :]
    s_ = sin[pos][:, :, None, :]
    mask = torch.arange(gen.max_seq, device=dev)[None, None, :] <= pos[:, :, None]
    bidx = torch.arange(B, device=dev)[:, None]
    h, rows = decoder.decode_step_begin(tok.reshape(B), pos.reshape(B), model.tok_embeddings.weight, cos, sin)
    assert torch.equal(h, model.tok_embeddings(tok.reshape(B)))
    hc = h.clone()  # the glue path's own chain
    worst = {"bitlinear": 0.0, "attention_abs": 0.0, "layer": 0.0}

    def sub(name, li, got, want):
        r = _rel_l2(got, want)
        worst["bitlinear"] = max(worst["bitlinear"], r)
        assert r <= 2.0 ** -8, f"layer {li} {name}: relative L2 distance {r}"

    def glue_attention(att, x, ck, cv):
        gk, gv = ck.clone(), cv.clone()
        q, k, v = att.split_qkv(x[:, None, :])
        q, k = decoder.apply_rope(q, c, s_), decoder.apply_rope(k, c, s_)
        gk.index_put_((bidx, pos), k)
        gv.index_put_((bidx, pos), v)
        return att.attend(q, gk, gv, mask)[:, 0], gk, gv

    for li, (layer, (ck, cv)) in enumerate(zip(model.layers, gen.cache)):
        att, ffn = layer.attention, layer.feed_forward
        # the glue path's own chain first (cache copies)
        o_c, _, _ = glue_attention(att, att.wqkv(layer.attention_norm(hc)), ck, cv)
        hc1 = hc + att.wo(att.attn_sub_norm(o_c))
        hc = hc1 + ffn(layer.ffn_norm(hc1))
        # fused sub-steps, each against the glue evaluation of the same input
        h_in = h
        xqkv = decoder.norm_bitlinear(h, layer.attention_norm, att.wqkv)
        sub("wqkv", li, xqkv, att.wqkv(layer.attention_norm(h)))
        o_g, gk, gv = glue_attention(att, xqkv, ck, cv)
        o_f = decoder.attn_decode(xqkv, ck, cv, pos.reshape(B), cos, sin, a.n_heads, a.n_kv_heads, gen.attn_ws, rope_rows=rows)
        assert torch.equal(ck, gk) and torch.equal(cv, gv), f"layer {li}: cache rows"
        bad = (_ulp(o_f, o_g) > 3) & ((o_f.float() - o_g.float()).abs() > 4e-3)
        worst["attention_abs"] = max(worst["attention_abs"], float((o_f.float() - o_g.float()).abs().max()))
        assert not bad.any(), f"layer {li} attention: {int(bad.sum())} of {bad.numel()} outside tolerance"
        h1 = decoder.norm_bitlinear(o_f, att.attn_sub_norm, att.wo, residual=h)
        sub("wo + residual", li, h1, h + att.wo(att.attn_sub_norm(o_f)))
        x13 = decoder.norm_bitlinear(h1, layer.ffn_norm, ffn.w13)
        sub("w13", li, x13, ffn.w13(layer.ffn_norm(h1)))
        h = decoder.norm_bitlinear(x13, ffn.ffn_sub_norm, ffn.w2, glu=True, residual=h1)
        x1, x3 = x13.chunk(2, -1)
        sub("w2 + residual", li, h, h1 + ffn.w2(ffn.ffn_sub_norm(torch.relu(x1) ** 2 * x3)))
        # the whole glue layer on the fused layer's input, for the record
        o_l, _, _ = glue_attention(att, att.wqkv(layer.attention_norm(h_in)), ck, cv)
        hl = h_in + att.wo(att.attn_sub_norm(o_l))
        hl = hl + ffn(layer.ffn_norm(hl))
        worst["layer"] = max(worst["layer"], _rel_l2(h, hl))
    gen.attn_ws.check()
    return h, hc, worst


@pytest.mark.parametrize("B", [1, 8])
def test_full_size_decode_step_substeps_against_the_torch_glue(model_2b, B):
    """Position 512 of the full-size model after the 512-token prompt: all 30 x 5
    sub-steps of the fused decode step against the torch glue on identical
    inputs (bounds: see _decode_step_substeps_against_glue), the library's LM head
    against the argmax of torch logits, and, end to end over the 30 layers, the
    two paths' logits still pointing the same way (cosine above 0.9: per layer the
    quantizers amplify the attention's rounding to 1-3 %, see above)."""
    P = 512
    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(4321 + B)
    prompt = torch.randint(0, model_2b.args.vocab_size, (B, P), generator=g, device=dev)
    gen = decoder.Generator(model_2b, B, P + 8)
    first = gen.prefill(prompt)
    h, hc, worst = _decode_step_substeps_against_glue(model_2b, gen, first.view(B, 1), P)
    logits_f = model_2b.output(model_2b.norm(h)).float()
    logits_g = model_2b.output(model_2b.norm(hc)).float()
    cosine = torch.nn.functional.cosine_similarity(logits_f, logits_g, dim=-1)
    print(f"full-size step, batch {B}: worst BitLinear sub-step relative L2 {worst['bitlinear']:.2e}, worst attention "
          f"|diff| {worst['attention_abs']:.2e}, worst whole-layer relative L2 {worst['layer']:.2e}, logits cosine "
          f"{float(cosine.min()):.4f}, relative L2 {_rel_l2(logits_f, logits_g):.3f}")
    assert float(cosine.min()) > 0.9
    # the library's LM head on the fused hidden state: its greedy token is the argmax of these logits
    tok_lib = decoder.lm_head_greedy(h, model_2b.norm, model_2b.output.weight, gen.lm_ws)
    top2 = torch.topk(logits_f, 2, dim=-1).values
    clear = (top2[:, 0] - top2[:, 1]) > 2e-2  # rows whose best logit is not a near tie
    assert torch.equal(tok_lib[clear], torch.argmax(logits_f, dim=-1)[clear])


def test_decoder_loaded_from_a_gguf_file_gives_the_same_logits(tmp_path):
    """A decoder written out as a GGUF file with I2_S projections (the CPU stack's format) and read back
    through the transcoder computes, prompt and decode step, what the original computes: the packed bytes,
    the scale slots and the norms survive the trip bit for bit, so the logits are equal."""
    from bitnet_amd import gguf

    model = _build(SMALL, seed=4)
    state = {k: v.detach().cpu() for k, v in model.state_dict().items()}
    path = str(tmp_path / "small.gguf")
    gguf.int2_state_to_gguf(state, SMALL, path, embed_dtype=torch.bfloat16)
    with gguf.GGUFReader(path) as r:
        args = gguf.model_args_from_gguf(r)
        back = gguf.gguf_to_int2_state(r)
    assert args == SMALL
    for k, v in state.items():
        assert torch.equal(back[k], v), k
    clone = _build(args, seed=9)  # other weights, then overwritten by the file's
    clone.load_state_dict(back, strict=True)
    B, P, S = 2, 20, 32
    dev = torch.device("cuda")
    cos, sin = decoder.rope_tables(SMALL.dim // SMALL.n_heads, S, SMALL.rope_theta, dev)
    g = torch.Generator(device="cuda").manual_seed(8)
    prompt = torch.randint(0, SMALL.vocab_size, (B, P), generator=g, device=dev)
    pos = torch.arange(P, device=dev)[None].expand(B, P).contiguous()
    c1, c2 = model.make_cache(B, S, dev), clone.make_cache(B, S, dev)
    l1 = model.forward_tokens(prompt, pos, c1, cos, sin)
    l2 = clone.forward_tokens(prompt, pos, c2, cos, sin)
    assert torch.equal(l1, l2) and bool(torch.isfinite(l1).all())
    tok = torch.argmax(l1[:, -1], dim=-1).view(B, 1)
    p1 = torch.full((B, 1), P, device=dev)
    assert torch.equal(model.forward_tokens(tok, p1, c1, cos, sin), clone.forward_tokens(tok, p1, c2, cos, sin))


def test_generate_all_with_ragged_prompts_equals_one_sequence_at_a_time():
    """FastGen.generate_all semantics (gpu/generate.py:217-304): prompts of different lengths in one batch,
    padded on the right.  Every per-token operation is independent of the other rows and the attention of a
    sequence only sees its own cache rows up to its own position, so each answer equals what the same prompt
    generates alone -- on the fused path (graph replays) and on the torch-glue path."""
    model = _build(BIG_HEADS, seed=5)
    assert decoder.Generator(model, batch=3, max_seq=64).lm_head  # head_dim 128: the folded calls and the library's LM head
    g = torch.Generator().manual_seed(3)
    prompts = [torch.randint(2, BIG_HEADS.vocab_size, (n,), generator=g).tolist() for n in (19, 7, 33)]
    gen = 12
    for fused in (True, False):
        batch = decoder.Generator(model, batch=3, max_seq=64, use_graph=fused, fused=fused)
        answers = batch.generate_all(prompts, gen)
        assert [len(a) for a in answers] == [gen] * 3
        for b, q in enumerate(prompts):
            alone = decoder.Generator(model, batch=1, max_seq=64, use_graph=fused, fused=fused)
            assert alone.generate_all([q], gen) == [answers[b]], (fused, b)
    with pytest.raises(ValueError):
        batch.generate_all(prompts[:2], gen)
    with pytest.raises(ValueError):
        batch.generate_all(prompts, 64)
    with pytest.raises(ValueError):
        batch.generate_all([[BIG_HEADS.vocab_size], [1], [1]], 4)


def test_generate_all_stops_at_the_end_token_and_trims_the_answers():
    model = _build(BIG_HEADS, seed=6)
    g = torch.Generator().manual_seed(4)
    prompts = [torch.randint(2, BIG_HEADS.vocab_size, (n,), generator=g).tolist() for n in (9, 14)]
    gen = decoder.Generator(model, batch=2, max_seq=48)
    full = gen.generate_all(prompts, 16)
    # take a token that sequence 1 produces at step 5 as the end token
    eos = full[1][5]
    # the loop ends after the first DECODE step (index >= 1) in which any sequence produced it: a hit in the
    # prompt pass's own token does not end the batch (gpu/generate.py:262-284)
    first_hit = min([a.index(eos, 1) for a in full if eos in a[1:]] + [15])
    timings = {}
    cut = gen.generate_all(prompts, 16, eos_id=eos, timings=timings)
    assert timings["decode_tokens"] == 2 * (len(max(cut, key=len)) - 1) or timings["decode_tokens"] == 2 * first_hit
    assert timings["prefill_s"] > 0 and timings["decode_s"] > 0 and timings["decode_tokens_per_s"] > 0
    for a, f in zip(cut, full):
        want = f[: first_hit + 1]           # the loop ends after the first step in which any sequence hit it
        if eos in want:
            want = want[: want.index(eos) + 1]
        assert a == want
    assert cut[1][-1] == eos or eos in cut[0]
    # the end token as the very first token of sequence 0 (out of the prompt pass): that sequence's answer is the end
    # token alone, the other sequence goes on as if nothing had happened, until a decode step produces the token
    eos0 = full[0][0]
    cut0 = gen.generate_all(prompts, 16, eos_id=eos0)
    assert cut0[0] == [eos0]
    hit = min([a.index(eos0, 1) for a in full if eos0 in a[1:]] + [15])
    want1 = full[1][: hit + 1]
    if eos0 in want1:
        want1 = want1[: want1.index(eos0) + 1]
    assert cut0[1] == want1 and len(cut0[1]) > 1


def test_generate_all_sampling_is_reproducible_and_greedy_for_a_tiny_nucleus():
    model = _build(BIG_HEADS, seed=7)
    g = torch.Generator().manual_seed(5)
    prompts = [torch.randint(2, BIG_HEADS.vocab_size, (n,), generator=g).tolist() for n in (11, 6)]
    gen = decoder.Generator(model, batch=2, max_seq=40)
    a = gen.generate_all(prompts, 10, use_sampling=True, rng=torch.Generator(device="cuda").manual_seed(11))
    b = gen.generate_all(prompts, 10, use_sampling=True, rng=torch.Generator(device="cuda").manual_seed(11))
    c = gen.generate_all(prompts, 10, use_sampling=True, rng=torch.Generator(device="cuda").manual_seed(12))
    assert a == b and all(0 <= t < BIG_HEADS.vocab_size for ans in a for t in ans)
    assert a != c  # 20 draws at temperature 0.7 from a 512-token vocabulary
    # a nucleus that only holds the most likely token: the greedy answer (the draw is from the bf16-rounded
    # logits the LM head returns, the greedy token from the same values)
    greedy = gen.generate_all(prompts, 10)
    tiny = gen.generate_all(prompts, 10, use_sampling=True, top_p=1e-9, rng=torch.Generator(device="cuda").manual_seed(1))
    assert tiny == greedy


def test_captured_prompt_pass_equals_the_launch_by_launch_one():
    """Generator.prefill replays one captured graph per bucket of prompt lengths (multiples of 32 tokens, the
    prompt padded up to the bucket); every replay, with other work of the program in between (decode steps,
    prompts of other lengths), gives the tokens, and leaves the cache rows, of the unpadded pass issued launch by
    launch.  Beyond kMaxPrefillGraphs captured passes the least recently used one is dropped."""
    model = _build(BIG_HEADS, seed=8)
    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(21)
    graphed = decoder.Generator(model, batch=2, max_seq=96, use_graph=True)
    eager = decoder.Generator(model, batch=2, max_seq=96, use_graph=False)
    assert graphed.lm_head and eager.lm_head
    for rnd, P in enumerate((24, 40, 24, 24, 7, 40)):
        prompt = torch.randint(0, BIG_HEADS.vocab_size, (2, P), generator=g, device=dev)
        t1 = graphed.prefill(prompt)
        t2 = eager.prefill(prompt)
        assert torch.equal(t1, t2), (rnd, P)
        for (k1, v1), (k2, v2) in zip(graphed.cache, eager.cache):
            assert torch.equal(k1[:, :P], k2[:, :P]) and torch.equal(v1[:, :P], v2[:, :P])
        # the program's own work between two replays
        d1 = graphed.decode(t1, P, 5)
        d2 = eager.decode(t2, P, 5)
        assert torch.equal(d1, d2)
    assert sorted(k[0] for k in graphed._pf_graphs) == [32, 64]  # 7 and 24 share a pass, 40 has the other
    # a bucket cut short by the cache's capacity, and the bound on the passes kept
    graphed.kMaxPrefillGraphs = 2
    prompt = torch.randint(0, BIG_HEADS.vocab_size, (2, 70), generator=g, device=dev)
    assert torch.equal(graphed.prefill(prompt), eager.prefill(prompt))
    assert [k[0] for k in graphed._pf_graphs] == [64, 96]  # 32, replayed longest ago, made room
    prompt = torch.randint(0, BIG_HEADS.vocab_size, (2, 9), generator=g, device=dev)
    assert torch.equal(graphed.prefill(prompt), eager.prefill(prompt))
    assert [k[0] for k in graphed._pf_graphs] == [96, 32]
    graphed.kMaxPrefillGraphs = 12
    # ragged prompts go through the same captured pass with their own lengths
    prompts = [torch.randint(2, BIG_HEADS.vocab_size, (n,), generator=torch.Generator().manual_seed(n)).tolist() for n in (40, 13)]
    assert graphed.generate_all(prompts, 6) == eager.generate_all(prompts, 6)
    prompts = [prompts[1], prompts[0]]
    assert graphed.generate_all(prompts, 6) == eager.generate_all(prompts, 6)


# ---------------------------------------------------------------------------
# A converted Hugging Face checkpoint through the decoder (gpu/convert_safetensors.py:43-93,
# gpu/convert_checkpoint.py:29-32, 42-77)
# ---------------------------------------------------------------------------
HF_ARGS = decoder.ModelArgs(dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=320, ffn_dim=768, segment_scales=True)


def _hf_checkpoint(args, seed):
    """Synthetic tensors under the Hugging Face names, bf16 like the published master weights; q, k and v
    projections of clearly different magnitude, so that their three weight scales differ by factors."""
    g = torch.Generator().manual_seed(seed)
    hd = args.dim // args.n_heads
    r = lambda std, *shape: (torch.randn(*shape, generator=g) * std).to(torch.bfloat16)
    st = {}
    for layer in range(args.n_layers):
        b = f"model.layers.{layer}."
        st[b + "self_attn.q_proj.weight"] = r(0.02, args.n_heads * hd, args.dim)
        st[b + "self_attn.k_proj.weight"] = r(0.06, args.n_kv_heads * hd, args.dim)
        st[b + "self_attn.v_proj.weight"] = r(0.009, args.n_kv_heads * hd, args.dim)
        st[b + "self_attn.o_proj.weight"] = r(0.02, args.dim, args.n_heads * hd)
        st[b + "input_layernorm.weight"] = 1 + r(0.1, args.dim)
        st[b + "post_attention_layernorm.weight"] = 1 + r(0.1, args.dim)
        st[b + "self_attn.attn_sub_norm.weight"] = 1 + r(0.1, args.dim)
        st[b + "mlp.ffn_sub_norm.weight"] = 1 + r(0.1, args.ffn_dim)
        st[b + "mlp.gate_proj.weight"] = r(0.03, args.ffn_dim, args.dim)
        st[b + "mlp.up_proj.weight"] = r(0.015, args.ffn_dim, args.dim)
        st[b + "mlp.down_proj.weight"] = r(0.02, args.dim, args.ffn_dim)
    st["model.embed_tokens.weight"] = r(0.5, args.vocab_size, args.dim)
    st["model.norm.weight"] = 1 + r(0.1, args.dim)
    return st


def _hf_convention_logits(st, args, ids):
    """The model the checkpoint describes, evaluated the way the Hugging Face side of the reference's converter
    sees it, in plain torch: projections kept apart and in their original row order, rotary embedding on the two
    halves of a head (rotate_half), every BitLinear as the reference's fp module (activations snapped to the int8
    grid, gpu/model.py:77-85, times weights ternarised and dequantised per tensor, gpu/convert_checkpoint.py:29-32),
    sub-norms and squared-ReLU gate as gpu/model.py:159-160, 195-196.  fp32 arithmetic, rounded to bf16 where the
    decoder's tensors are bf16.  ids [B, T] -> logits fp32 [B, T, vocab]."""
    dev = ids.device
    bf = torch.bfloat16
    hd = args.dim // args.n_heads
    rep = args.n_heads // args.n_kv_heads
    B, T = ids.shape
    w = {k: v.to(dev) for k, v in st.items()}

    def rms(x, g):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + args.norm_eps) * g.float()).to(bf)

    def deq(t):  # convert_checkpoint.py:29-32, in the checkpoint's dtype
        s = 1.0 / t.abs().mean().clamp_(min=1e-5)
        return ((t * s).round().clamp(-1, 1) / s).float()

    def bitlinear_fp(x, t):  # gpu/model.py:77-85
        xf = x.float()
        s = 127 / xf.abs().max(dim=-1, keepdim=True).values.clamp_(min=1e-5)
        return (((xf * s).round().clamp(-128, 127) / s) @ deq(t).T).to(bf)

    inv = 1.0 / (args.rope_theta ** (torch.arange(0, hd, 2, device=dev, dtype=torch.float32) / hd))
    ang = torch.outer(torch.arange(T, device=dev, dtype=torch.float32), inv)
    cos = torch.cat([ang.cos(), ang.cos()], dim=-1)[None, :, None, :]  # [1, T, 1, hd]: frequency i at i and i + hd/2
    sin = torch.cat([ang.sin(), ang.sin()], dim=-1)[None, :, None, :]

    def rope_half(x):  # x [B, T, heads, hd]
        xf = x.float()
        x1, x2 = xf[..., : hd // 2], xf[..., hd // 2 :]
        return (xf * cos + torch.cat([-x2, x1], dim=-1) * sin).to(bf)

    h = w["model.embed_tokens.weight"][ids]  # [B, T, dim] bf16
    causal = torch.ones(T, T, dtype=torch.bool, device=dev).tril()
    for layer in range(args.n_layers):
        b = f"model.layers.{layer}."
        x = rms(h, w[b + "input_layernorm.weight"])
        q = rope_half(bitlinear_fp(x, w[b + "self_attn.q_proj.weight"]).view(B, T, args.n_heads, hd))
        k = rope_half(bitlinear_fp(x, w[b + "self_attn.k_proj.weight"]).view(B, T, args.n_kv_heads, hd))
        v = bitlinear_fp(x, w[b + "self_attn.v_proj.weight"]).view(B, T, args.n_kv_heads, hd)
        k = k.repeat_interleave(rep, dim=2).float()  # query head j reads kv head j // rep
        v = v.repeat_interleave(rep, dim=2).float()
        sc = torch.einsum("bthd,bshd->bhts", q.float(), k) * hd ** -0.5
        sc = sc.masked_fill(~causal[None, None], float("-inf"))
        o = torch.einsum("bhts,bshd->bthd", torch.softmax(sc, dim=-1), v).reshape(B, T, args.dim).to(bf)
        h = (h.float() + bitlinear_fp(rms(o, w[b + "self_attn.attn_sub_norm.weight"]), w[b + "self_attn.o_proj.weight"]).float()).to(bf)
        x = rms(h, w[b + "post_attention_layernorm.weight"])
        gate = bitlinear_fp(x, w[b + "mlp.gate_proj.weight"])
        up = bitlinear_fp(x, w[b + "mlp.up_proj.weight"])
        inner = ((torch.relu(gate.float()) ** 2).to(bf).float() * up.float()).to(bf)
        h = (h.float() + bitlinear_fp(rms(inner, w[b + "mlp.ffn_sub_norm.weight"]), w[b + "mlp.down_proj.weight"]).float()).to(bf)
    return rms(h, w["model.norm.weight"]).float() @ w["model.embed_tokens.weight"].float().T


def _load_converted(path, args):
    with torch.device("cuda"):
        prev = torch.get_default_dtype()
        torch.set_default_dtype(torch.bfloat16)
        try:
            model = decoder.Transformer(args)
        finally:
            torch.set_default_dtype(prev)
    model.load_state_dict(torch.load(path, weights_only=True), strict=True)
    return model


def test_converted_hf_checkpoint_runs_through_the_decoder_like_the_hf_convention_model(tmp_path):
    """Row (f3) on the device: synthetic Hugging Face tensors -> convert_hf_checkpoint (rotary row permutation,
    q|k|v and gate|up fusing, per-sub-tensor ternarisation, four-slot scales, packing) -> strict load into the
    decoder -> prompt pass and decode step through the library's int8 kernels with the segment scale rule.  The
    yardstick never sees a fused, permuted or packed tensor: it evaluates the unfused projections with half-split
    rotary embedding and the reference's fp BitLinear.  Attention scores are invariant under the permutation
    (q and k are permuted alike within a head), and the int8 path differs from the fp module only in where
    roundings fall (same integer products; tests/test_gpu_bitlinear.py::test_fp_path_agrees_with_the_int8_path
    derives the per-call bound), so the logits agree up to the amplification of those roundings by the later
    quantizers: a few percent of the logits' norm.  A wrong row order, segment boundary or scale slot moves them
    by tens of percent -- the control at the end runs the same file with the reference kernel's slot rule
    n // (N // ws_num) (bitnet_kernels.h:80; one slot for a shape outside its table, so k and v rows are scaled
    by s_q) and must land far outside the bound."""
    from safetensors.torch import save_file

    from bitnet_amd import checkpoint

    args = HF_ARGS
    st = _hf_checkpoint(args, seed=11)
    src = str(tmp_path / "model.safetensors")
    save_file(st, src)
    path = checkpoint.convert_hf_checkpoint(src, str(tmp_path / "out"), args)
    model = _load_converted(path, args)
    for lr in model.layers:  # the three scales of a fused wqkv really differ, else the control below proves nothing
        s3 = lr.attention.wqkv.weight_scale.float()
        assert float(s3[1] / s3[0]) > 2.0 and float(s3[0] / s3[2]) > 1.5 and float(s3[3]) == 0.0

    dev = torch.device("cuda")
    B, T, S = 2, 48, 64
    g = torch.Generator(device="cuda").manual_seed(12)
    ids = torch.randint(0, args.vocab_size, (B, T + 1), generator=g, device=dev)
    want = _hf_convention_logits(st, args, ids)  # [B, T + 1, V]

    @torch.no_grad()
    def run(m):
        cos, sin = decoder.rope_tables(args.dim // args.n_heads, S, args.rope_theta, dev)
        cache = m.make_cache(B, S, dev)
        hid = m.prefill_hidden_fused(ids[:, :T].contiguous(), cache, cos, sin)  # quantizer kernels + int8 MFMA GEMM
        prompt_logits = m.output(m.norm(hid)).float()
        ws = decoder.AttnWorkspace(B, args.n_heads, args.n_kv_heads, 8, dev)
        pos = torch.full((B, 1), T, device=dev)
        step_logits = m.forward_decode_fused(ids[:, T:].contiguous(), pos, cache, cos, sin, ws)  # one-kernel forwards
        ws.check()
        # the unfused glue (BitLinearKernel.forward per projection) on the same prompt
        glue = m.forward_tokens(ids[:, :T].contiguous(), torch.arange(T, device=dev)[None].expand(B, T).contiguous(),
                                m.make_cache(B, S, dev), cos, sin)
        torch.cuda.synchronize()
        return torch.cat([prompt_logits, step_logits], dim=1), glue

    rel = lambda a, b: float((a - b).norm() / b.norm())
    got, glue = run(model)
    assert bool(torch.isfinite(got).all())
    err_prompt, err_step, err_glue = rel(got[:, :T], want[:, :T]), rel(got[:, T:], want[:, T:]), rel(glue, want[:, :T])
    bound = 0.035  # measured 0.017-0.020 over three seeds
    assert err_prompt < bound and err_step < bound and err_glue < bound, (err_prompt, err_step, err_glue)
    top = want.topk(2, dim=-1).values
    clear = (top[..., 0] - top[..., 1]) > 0.15 * want.std()
    assert int(clear.sum()) > 10
    assert torch.equal(got.argmax(-1)[clear], want.argmax(-1)[clear])

    # control: the same file through the reference kernel's slot rule
    import dataclasses

    thirds = _load_converted(path, dataclasses.replace(args, segment_scales=False))
    got3, _ = run(thirds)
    assert rel(got3, want) > 2 * bound, rel(got3, want)  # measured 0.094-0.112

    # control: a converter that forgot the rotary row permutation of q and k (convert_safetensors.py:43-47)
    state = checkpoint.hf_to_model_state(st, args)
    hd = args.dim // args.n_heads
    for layer in range(args.n_layers):
        b = f"model.layers.{layer}.self_attn."
        state[f"layers.{layer}.attention.wqkv.weight"] = torch.cat(
            [st[b + "q_proj.weight"], st[b + "k_proj.weight"], st[b + "v_proj.weight"]], dim=0)
    bad = str(tmp_path / "unpermuted.pt")
    torch.save(checkpoint.model_state_to_int2(state, args), bad)
    got_bad, _ = run(_load_converted(bad, args))
    assert rel(got_bad, want) > 2 * bound, rel(got_bad, want)
