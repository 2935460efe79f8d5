"""CPU tests of the config-4 harness (dsaquant_amd/wan_harness.py): every piece the harness restates from the
reference's Wan DiT is held to a closed form or a torch primitive written out independently here, and the
30-layer model is built on the meta device through the packed loader and counted as the reference's build smoke
test counts it (tests/test_vdm_eval_build_smoke.py:15-25)."""
import math
from dataclasses import replace

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F
from einops import rearrange

from dsaquant_amd import wan_harness as W


def test_rope_frequencies_closed_form_with_the_44_42_42_split():
    """modules/embedding.py:114-157: head dim 128 splits into 44 channels for the frame index and 42 each for row and
    column; channel pair j of an axis with d channels turns by pos * 10000^(-2j/d)."""
    f, h, w, hd = 2, 3, 2, 128
    freqs = W.rope_frequencies(hd, f, h, w, "cpu")
    assert freqs.shape == (f * h * w, 1, hd // 2) and freqs.dtype == torch.complex64
    dims = (hd - 2 * (hd // 3), hd // 3, hd // 3)
    assert dims == (44, 42, 42)
    for fi in range(f):
        for hi in range(h):
            for wi in range(w):
                row = freqs[(fi * h + hi) * w + wi, 0]
                want = []
                for pos, d in zip((fi, hi, wi), dims):
                    want += [complex(math.cos(pos * 10000.0 ** (-2.0 * j / d)), math.sin(pos * 10000.0 ** (-2.0 * j / d))) for j in range(d // 2)]
                got = [complex(z) for z in row.tolist()]
                assert len(got) == len(want) == 64
                assert max(abs(a - b) for a, b in zip(got, want)) < 1e-6, (fi, hi, wi)


def test_apply_rope_is_a_rotation_of_consecutive_channel_pairs():
    """modules/attention.py:133-137: channels (2j, 2j+1) form the complex number that is multiplied by the position's
    unit complex; written out in real arithmetic here."""
    g = torch.Generator().manual_seed(0)
    f, h, w, heads, hd = 2, 2, 3, 3, 128
    L = f * h * w
    x = torch.randn((1, L, heads, hd), generator=g)
    freqs = W.rope_frequencies(hd, f, h, w, "cpu")
    got = W.apply_rope(x, freqs)
    cos, sin = freqs.real[:, 0].float(), freqs.imag[:, 0].float()  # [L, hd/2]
    even, odd = x[..., 0::2], x[..., 1::2]
    want = torch.empty_like(x)
    want[..., 0::2] = even * cos[None, :, None, :] - odd * sin[None, :, None, :]
    want[..., 1::2] = even * sin[None, :, None, :] + odd * cos[None, :, None, :]
    assert torch.allclose(got, want, atol=1e-6, rtol=0)
    # position 0 is the identity; norms of pairs are kept everywhere
    assert torch.allclose(got[:, 0], x[:, 0], atol=1e-7, rtol=0)
    assert torch.allclose(got[..., 0::2] ** 2 + got[..., 1::2] ** 2, even ** 2 + odd ** 2, atol=1e-5, rtol=1e-5)
    # fp16 in, fp16 out, arithmetic in fp32
    xh = x.half()
    assert W.apply_rope(xh, freqs).dtype == torch.float16
    assert torch.equal(W.apply_rope(xh, freqs), W.apply_rope(xh.float(), freqs).half())


def test_rms_norm_across_heads_against_torch():
    """modules/attention.py:208-216: x * rsqrt(mean(x^2) + eps) in fp32 over the FULL dim (all heads), cast back, then
    the weight."""
    g = torch.Generator().manual_seed(1)
    dim, eps = 384, 1e-6
    m = W.RMSNormAcrossHeads(dim, eps)
    with torch.no_grad():
        m.weight.copy_(torch.rand(dim, generator=g) + 0.5)
    x = torch.randn((2, 7, dim), generator=g)
    want = F.rms_norm(x.double(), (dim,), m.weight.double(), eps)
    assert torch.allclose(m(x).double(), want, atol=1e-5, rtol=1e-5)
    # not a per-head norm: scaling one head changes the others' outputs
    y = x.clone()
    y[..., :128] *= 3.0
    assert not torch.allclose(m(y)[..., 128:], m(x)[..., 128:], atol=1e-3)
    # fp16: normalise in fp32, round, multiply by the weight in the input dtype
    xh = x.half()
    mh = W.RMSNormAcrossHeads(dim, eps).half()
    with torch.no_grad():
        mh.weight.copy_(m.weight.half())
    xf = xh.float()
    want_h = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).half() * mh.weight
    assert torch.equal(mh(xh), want_h)


def test_fp32_layer_norm_against_float64_statistics():
    """diffusers' FP32LayerNorm as the blocks use it (dit_block.py:32, :52): statistics and affine in fp32 whatever
    the input dtype, result cast back."""
    g = torch.Generator().manual_seed(2)
    dim, eps = 256, 1e-6
    x = (torch.randn((3, 5, dim), generator=g) * 4 + 1).half()
    wt, b = torch.rand(dim, generator=g) + 0.5, torch.randn(dim, generator=g)
    xd = x.double()
    mean, var = xd.mean(-1, keepdim=True), xd.var(-1, unbiased=False, keepdim=True)
    plain = (xd - mean) / torch.sqrt(var + eps)
    got = W.fp32_layer_norm(x, None, None, eps)
    assert got.dtype == torch.float16
    assert (got.double() - plain).abs().max() <= 2.0 ** -10 * plain.abs().max()  # one fp16 rounding of values below 8
    got_affine = W.fp32_layer_norm(x, wt.half(), b.half(), eps)
    want_affine = plain * wt.half().double() + b.half().double()
    assert (got_affine.double() - want_affine).abs().max() <= 2.0 ** -10 * want_affine.abs().max()


def test_timestep_embedding_closed_form():
    """modules/embedding.py:7-10: [cos(t * 10000^(-i/128)) for i < 128] then the sines, float64."""
    t = torch.tensor([999.0, 428.0, 0.0])
    got = W.timestep_embedding(256, t)
    assert got.shape == (3, 256) and got.dtype == torch.float64
    for r, tv in enumerate(t.tolist()):
        for i in (0, 1, 17, 127):
            a = tv * 10000.0 ** (-i / 128.0)
            assert abs(got[r, i].item() - math.cos(a)) < 1e-9 and abs(got[r, 128 + i].item() - math.sin(a)) < 1e-9


def test_patchify_and_unpatchify_orders():
    """Input patches are channel-major ('1 c (f c1) (h c2) (w c3) -> 1 (f h w) (c c1 c2 c3)', modules/model.py:193-199);
    the head's output of a token is patch-position major ('1 l (n c) -> 1 (l n) c', n = 4, modules/model.py:353)."""
    with torch.device("meta"):
        m = W.WanDiT(replace(W.WAN21_1P3B, num_layers=1))
    x = torch.arange(16 * 3 * 8 * 12, dtype=torch.float32).reshape(1, 16, 3, 8, 12)
    tok = m.patchify(x)
    assert tok.shape == (1, 3 * 4 * 6, 64)
    assert torch.equal(tok, rearrange(x, "1 c (f c1) (h c2) (w c3) -> 1 (f h w) (c c1 c2 c3)", c1=1, c2=2, c3=2))
    assert tok[0, 0, 5].item() == x[0, 1, 0, 0, 1].item()  # element [c, dh, dw] at index c*4 + dh*2 + dw
    head = torch.arange(72 * 64, dtype=torch.float32).reshape(1, 72, 64)
    per_patch_position = rearrange(head, "1 l (n c) -> 1 (l n) c", n=4)  # the reference's output form
    want = rearrange(per_patch_position, "1 (f h w c2 c3) c -> 1 c f (h c2) (w c3)", f=3, h=4, w=6, c2=2, c3=2)
    assert torch.equal(m.unpatchify(head, 3, 8, 12), want)


def _reference_block(block: W.Block, x, context, tproj, freqs):
    """dit_block.py:96-114 written out with the reference's own rearrange + chunk, the block's sub-modules as they
    are."""
    table = block.scale_shift_table.to(tproj.dtype) + tproj
    shift_msa, scale_msa, gate_msa, c_shift_msa, c_scale_msa, c_gate_msa = rearrange(table, "l n c -> n l c").chunk(6, dim=0)
    norm = lambda t: F.layer_norm(t.float(), (t.shape[-1],), None, None, block.eps).to(t.dtype)  # noqa: E731
    h = norm(x) * (1 + scale_msa) + shift_msa
    x = x + block.attn1(h, None, freqs) * gate_msa
    h = F.layer_norm(x.float(), (x.shape[-1],), block.norm2.weight.float(), block.norm2.bias.float(), block.eps).to(x.dtype)
    x = x + block.attn2(h, context, None)
    h = norm(x) * (1 + c_scale_msa) + c_shift_msa
    return x + block.ffn(h) * c_gate_msa


def test_block_follows_the_adaln_chunk_order():
    """shift, scale, gate of the self-attention, then shift, scale, gate of the FFN (dit_block.py:96-100): the block
    with plain Linear layers against the sequence written out above; a swapped pair of rows must show."""
    torch.manual_seed(3)
    a = replace(W.WAN21_1P3B, num_layers=1, num_heads=2, ffn_dim=512)
    blk = W.Block(a).float()
    with torch.no_grad():
        blk.norm2.weight.uniform_(0.5, 1.5)
        blk.norm2.bias.normal_()
    f, h, w = 1, 2, 3
    x = torch.randn(1, f * h * w, a.dim)
    ctx = torch.randn(1, 5, a.dim)
    tproj = torch.randn(1, 6, a.dim)
    freqs = W.rope_frequencies(a.head_dim, f, h, w, "cpu")
    with torch.no_grad():
        got = blk(x, ctx, tproj, freqs)
        want = _reference_block(blk, x, ctx, tproj, freqs)
        assert torch.allclose(got, want, atol=1e-5, rtol=1e-5)
        swapped = _reference_block(blk, x, ctx, tproj[:, [1, 0, 2, 3, 4, 5]] + blk.scale_shift_table[:, [1, 0, 2, 3, 4, 5]]
                                   - blk.scale_shift_table, freqs)
        assert not torch.allclose(got, swapped, atol=1e-3)


def test_attention_module_against_written_out_sequence():
    """modules/attention.py:149-205: projections, RMS-norm of q and k across the full dim, heads split, RoPE on q and
    k of the self-attention only, mask-free SDPA, output projection."""
    torch.manual_seed(4)
    dim, heads = 256, 2
    att = W.Attention(dim, heads, 1e-6, cross=False).float()
    with torch.no_grad():
        att.norm_q.weight.uniform_(0.5, 1.5)
        att.norm_k.weight.uniform_(0.5, 1.5)
    f, h, w = 1, 2, 2
    x = torch.randn(1, f * h * w, dim)
    ctx = torch.randn(1, 3, dim)
    freqs = W.rope_frequencies(dim // heads, f, h, w, "cpu")

    def written_out(x, context, freqs):
        src = x if context is None else context
        q, k, v = att.to_q(x), att.to_k(src), att.to_v(src)
        q = F.rms_norm(q, (dim,), att.norm_q.weight, 1e-6)
        k = F.rms_norm(k, (dim,), att.norm_k.weight, 1e-6)
        q, k, v = (t.unflatten(2, (heads, -1)) for t in (q, k, v))
        if freqs is not None:
            q = torch.view_as_real(torch.view_as_complex(q.reshape(*q.shape[:-1], -1, 2)) * freqs).flatten(3)
            k = torch.view_as_real(torch.view_as_complex(k.reshape(*k.shape[:-1], -1, 2)) * freqs).flatten(3)
        scores = torch.einsum("blhd,bmhd->bhlm", q, k) / math.sqrt(dim // heads)
        o = torch.einsum("bhlm,bmhd->blhd", scores.softmax(-1), v).flatten(2, 3)
        return att.to_out[0](o)

    with torch.no_grad():
        assert torch.allclose(att(x, None, freqs), written_out(x, None, freqs), atol=1e-5, rtol=1e-5)
        assert torch.allclose(att(x, ctx, None), written_out(x, ctx, None), atol=1e-5, rtol=1e-5)


def _meta_packed_checkpoint(model):
    """A packed checkpoint of meta tensors with the shapes the loader expects."""
    from dsaquant_amd.checkpoints import packed_checkpoint as pc
    from dsaquant_amd.quantization.quant_linear import QuantLinear

    quant = {name: m for name, m in model.named_modules() if isinstance(m, QuantLinear)}
    sd = {}
    for key, p in model.state_dict().items():
        owner = key.rsplit(".", 1)[0]
        if ".wquantizer." in key or ".aquantizer." in key or (owner in quant and key.endswith(".weight")):
            continue
        sd[key] = torch.empty(p.shape, dtype=torch.float16, device="meta")
    for name, m in quant.items():
        n, k = m.out_features, m.in_features
        sd[f"{name}.vdm_weight_packed"] = torch.empty((n, k // 2), dtype=torch.uint8, device="meta")
        sd[f"{name}.vdm_weight_scale_packed"] = torch.empty((n, k // 64), dtype=torch.float16, device="meta")
        sd[f"{name}.vdm_weight_scale"] = torch.empty((n,), dtype=torch.float16, device="meta")
    return {"format": pc.PACKED_CHECKPOINT_FORMAT, "metadata": {}, "model": sd}


@pytest.mark.parametrize("args,layers,quant,attn", [(W.WAN21_1P3B, 30, 300, 60), (W.WAN21_14B, 40, 400, 80)])
def test_full_depth_model_counts_on_the_meta_device(args, layers, quant, attn):
    """What the reference's build smoke test prints for the quantized Wan-2.1 1.3B model
    (tests/test_vdm_eval_build_smoke.py:15-25): 300 QuantLinear layers, all in kernel mode, 60 attention modules, all
    on the fused vdm QKV path; 10 QuantLinear per block."""
    from dsaquant_amd.checkpoints import packed_checkpoint as pc
    from dsaquant_amd.quantization.quant_linear import QuantLinear

    assert args.num_layers == layers
    with torch.device("meta"):
        model = W.WanDiT(args)
    assert W.swap_block_linears(model) == quant
    missing, unexpected = pc.load_packed_quantized_model(model, _meta_packed_checkpoint(model), quant_linear_cls=QuantLinear,
                                                        dtype=torch.float16, device=torch.device("meta"), require_vdm_kernel=False)
    assert missing == [] and unexpected == []
    pc.enable_fused_qkv(model, quant_linear_cls=QuantLinear, attention_cls=W.Attention, use_fused_qkv=True)
    ql = [m for m in model.modules() if isinstance(m, QuantLinear)]
    assert len(ql) == quant and all(m.use_vdm_kernel for m in ql) and all(m.weight is None for m in ql)
    attns = [m for m in model.modules() if isinstance(m, W.Attention)]
    assert len(attns) == attn
    assert all(m.use_fused_qkv_kernel and m.qkv_kernel_backend == "vdm" for m in attns)
    assert not any(isinstance(m, QuantLinear) for m in (model.patch_embedding_mlp, model.proj_out, model.time_proj))
    for blk in model.blocks:
        assert sum(isinstance(m, QuantLinear) for m in blk.modules()) == 10
    # shapes of the W4A4 calls a block makes: fused q|k|v, attn1 out, attn2 q, attn2 k|v, attn2 out, FFN up, FFN down
    b = model.blocks[0]
    d = args.dim
    assert [tuple(l.vdm_weight_packed.shape) for l in (b.attn1.to_q, b.attn1.to_out[0], b.attn2.to_k, b.ffn.up, b.ffn.down)] == \
        [(d, d // 2), (d, d // 2), (d, d // 2), (args.ffn_dim, d // 2), (d, args.ffn_dim // 2)]
