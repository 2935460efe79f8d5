"""Minimal Wan DiT forward used as the caller-side harness of the W4A4 path.

This is NOT the reference's model code: it is a small restatement of the parts
of the Wan 2.1 transformer that decide WHICH W4A4 calls are made, with what
shapes, and what runs between them, so that the share of a denoise step spent
in the W4A4 kernels can be measured with random-init packed weights.  What it
reproduces, with the reference lines it follows:

* block structure (vdm_infer/models/wan_vdm/modules/dit_block.py:83-117):
  fp32 LayerNorm -> adaLN modulation -> self-attention (fused QKV) -> gated
  residual; affine fp32 LayerNorm -> cross-attention (to_q on the tokens, fused
  K|V on the 512 text tokens) -> residual; fp32 LayerNorm -> modulation ->
  GELU-tanh FFN -> gated residual.  Every Linear inside a block is a
  QuantLinear (10 per block, 7 W4A4 calls per block);
* attention (modules/attention.py:149-205): q/k RMS-norm across the full dim,
  complex interleaved-pair RoPE with the (44, 42, 42) split of head dim 128
  (modules/embedding.py:114-157), mask-free SDPA (models/base/vdm_attn.py:241-259);
* embeddings (modules/embedding.py:7-112): sinusoidal timestep -> MLP ->
  6*dim modulation, text MLP 4096 -> dim, patch MLP 64 -> dim; output head
  (modules/model.py:271-291);
* sequence mode: a forward sees one [1, L, C] token sequence
  (modules/model.py:192-202);
* the denoise loop's control flow (pipelines/text2video.py:522-609): a cond
  forward per step, an uncond forward when the active guidance scale is > 1,
  and the guidance scale switching to ``guidance_scale_2`` once
  t < boundary_ratio * 1000 (CFG-drop).  The scheduler is replaced by a plain
  Euler update (it is CPU scalar math plus one elementwise op per step).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from .checkpoints import packed_checkpoint as pc
from .fused_qkv import get_qkv_projections
from .quantization.quant_linear import QuantLinear


@dataclass
class WanArgs:
    """Hyper-parameters (vdm_infer/models/wan_vdm/__init__.py:13-31 for Wan-2.1 1.3B)."""
    num_layers: int = 30
    num_heads: int = 12
    head_dim: int = 128
    ffn_dim: int = 8960
    in_channels: int = 16
    text_dim: int = 4096
    freq_dim: int = 256
    patch_size: Tuple[int, int, int] = (1, 2, 2)
    eps: float = 1e-6

    @property
    def dim(self) -> int:
        return self.num_heads * self.head_dim


WAN21_1P3B = WanArgs()
WAN21_14B = WanArgs(num_layers=40, num_heads=40, ffn_dim=13824)


def fp32_layer_norm(x: torch.Tensor, weight, bias, eps: float) -> torch.Tensor:
    return F.layer_norm(x.float(), (x.shape[-1],), None if weight is None else weight.float(),
                        None if bias is None else bias.float(), eps).to(x.dtype)


class RMSNormAcrossHeads(nn.Module):
    def __init__(self, dim: int, eps: float):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + self.eps)).to(x.dtype) * self.weight


def rope_frequencies(head_dim: int, f: int, h: int, w: int, device) -> torch.Tensor:
    """complex64 [f*h*w, 1, head_dim/2]: frames get head_dim - 2*(head_dim//3) channels, rows and columns head_dim//3 each."""
    def axis(dim: int, n: int) -> torch.Tensor:
        freqs = 1.0 / (10000.0 ** (torch.arange(0, dim, 2)[: dim // 2].double() / dim))
        ang = torch.outer(torch.arange(n), freqs)
        return torch.polar(torch.ones_like(ang), ang)

    d3 = head_dim // 3
    ff, hh, ww = axis(head_dim - 2 * d3, f), axis(d3, h), axis(d3, w)
    freqs = torch.cat([ff.view(f, 1, 1, -1).expand(f, h, w, -1), hh.view(1, h, 1, -1).expand(f, h, w, -1),
                       ww.view(1, 1, w, -1).expand(f, h, w, -1)], dim=-1)
    return freqs.reshape(f * h * w, 1, -1).to(torch.complex64).to(device)


def timestep_embedding(freq_dim: int, timestep: torch.Tensor) -> torch.Tensor:
    """[B] -> [B, freq_dim] in float64: cos of the freq_dim/2 angles t * 10000^(-i / (freq_dim/2)) first, then their
    sin (modules/embedding.py:7-10)."""
    half = freq_dim // 2
    ang = torch.outer(timestep.double(), torch.pow(10000.0, -torch.arange(half, dtype=torch.float64, device=timestep.device) / half))
    return torch.cat([torch.cos(ang), torch.sin(ang)], dim=1)


def apply_rope(x: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """x [B, L, H, D]; consecutive channel pairs are rotated (fp32 complex arithmetic)."""
    xc = torch.view_as_complex(x.float().reshape(*x.shape[:-1], -1, 2))
    return torch.view_as_real(xc * freqs).flatten(3).to(x.dtype)


class SharedContext:
    """The cross-attention context of one forward together with its per-token quantization, made once per clip
    ratio and read by every block's K/V projection (the reference quantizes it in each block, dit_block.py:109)."""

    def __init__(self, tensor: torch.Tensor):
        self.tensor = tensor
        self._quantized = {}

    def quantized(self, clip_ratio: float):
        from . import fused_ops

        q = self._quantized.get(float(clip_ratio))
        if q is None:
            q = self._quantized[float(clip_ratio)] = fused_ops.QuantizedInput(self.tensor, clip_ratio)
        return q


def _version_of(tensor: torch.Tensor):
    return None if tensor.is_inference() else tensor._version


def _weak_lookup(cache: dict, tensor: torch.Tensor):
    # A tensor made under torch.inference_mode() counts no versions (reading the counter raises) yet can still be
    # written in place there, so nothing derived from one is reused: such a tensor is always a miss.
    if tensor.is_inference():
        return None
    hit = cache.get(id(tensor))
    if hit is not None and hit[0]() is tensor and hit[1] == _version_of(tensor):
        return hit[2]
    return None


def _weak_store(cache: dict, tensor: torch.Tensor, value) -> None:
    import weakref

    key = id(tensor)
    cache[key] = (weakref.ref(tensor, lambda _, d=cache, k=key: d.pop(k, None)), _version_of(tensor), value)


class Attention(nn.Module):
    def __init__(self, dim: int, heads: int, eps: float, cross: bool):
        super().__init__()
        self.heads = heads
        self.cross_attention_dim_head = dim // heads if cross else None
        self.to_q, self.to_k, self.to_v = nn.Linear(dim, dim), nn.Linear(dim, dim), nn.Linear(dim, dim)
        self.to_out = nn.ModuleList([nn.Linear(dim, dim)])
        self.norm_q, self.norm_k = RMSNormAcrossHeads(dim, eps), RMSNormAcrossHeads(dim, eps)
        self.fused_projections = False
        self.use_fused_qkv_kernel = False
        self.qkv_kernel_backend = None
        # q, k and v leave the fused GEMM as three contiguous tensors (the default, as in the reference, is three
        # strided views of one [tokens, 3 * dim] tensor): rotary embedding and SDPA then read contiguous rows
        self.qkv_contiguous_outputs = True
        self._cross_kv = {}

    # Cross-attention K (after norm_k) and V depend on the context only, which is the same tensor in every denoise
    # step of a prompt: keep them per context tensor (held weakly: a new tensor at a recycled address is a miss).
    cache_cross_kv = False

    def _context_kv(self, context):
        """K (normalised) and V of the cross-attention context, a tensor or a SharedContext."""
        from . import fused_ops

        tensor = context.tensor if isinstance(context, SharedContext) else context
        if self.cache_cross_kv:
            hit = _weak_lookup(self._cross_kv, tensor)
            if hit is not None:
                return hit
        kernel = getattr(self.to_k, "use_vdm_kernel", False)
        if kernel and isinstance(context, SharedContext):
            k, v = fused_ops.kv_projections(self, context.quantized(self.to_k.kernel_clip_ratio))
        elif kernel and self.use_fused_qkv_kernel:
            k, v = fused_ops.kv_projections(self, tensor)
        else:
            k, v = self.to_k(tensor), self.to_v(tensor)
        k = self.norm_k(k)
        if self.cache_cross_kv:
            _weak_store(self._cross_kv, tensor, (k, v))
        return k, v

    def forward(self, x, context: Optional[torch.Tensor], freqs: Optional[torch.Tensor], timers=None, residual=None, gate=None) -> torch.Tensor:
        """Returns the attention output, or ``residual + output * gate`` when ``residual`` is given (the update
        then runs in the output projection's GEMM epilogue if that projection is in kernel mode)."""
        from . import fused_ops

        if context is not None and (self.cache_cross_kv or isinstance(context, SharedContext)):
            tq = self.to_q
            if isinstance(x, fused_ops.LnInput):
                q = fused_ops.linear_ln_vdm_w4a4(x, tq.vdm_weight_packed, tq.vdm_weight_scale_packed, tq.bias, tq.kernel_clip_ratio,
                                                 bias_half=tq._bias_half)
            else:
                q = tq(x)
            q = self.norm_q(q)
            k, v = self._context_kv(context)
        else:
            if isinstance(x, fused_ops.LnInput):  # the LayerNorm in front of this module runs inside the quantizer
                if context is None:
                    q, k, v = fused_ops.qkv_projections_ln(self, x)
                else:
                    tq = self.to_q
                    q = fused_ops.linear_ln_vdm_w4a4(x, tq.vdm_weight_packed, tq.vdm_weight_scale_packed, tq.bias, tq.kernel_clip_ratio,
                                                     bias_half=tq._bias_half)
                    k, v = fused_ops.kv_projections(self, context)
            else:
                q, k, v = get_qkv_projections(self, x, context)
            q, k = self.norm_q(q), self.norm_k(k)
        q, k, v = (t.unflatten(2, (self.heads, -1)) for t in (q, k, v))
        if freqs is not None:
            q, k = apply_rope(q, freqs), apply_rope(k, freqs)
        if timers is not None:
            timers.start("attention")
        o = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), dropout_p=0.0, is_causal=False)
        if timers is not None:
            timers.stop("attention")
        return _project_and_update(self.to_out[0], o.transpose(1, 2).flatten(2, 3), None, residual, gate)


def _project_and_update(layer, y: torch.Tensor, act: Optional[str], residual, gate) -> torch.Tensor:
    """``residual + layer(act(y)) * gate`` -- in one fused linear when ``layer`` is a QuantLinear in kernel mode and
    something can be fused, otherwise as separate tensor operations (dit_block.py:102, :107, :112)."""
    if getattr(layer, "use_vdm_kernel", False) and (act is not None or residual is not None):
        from . import fused_ops

        return fused_ops.linear_fused(y, layer.vdm_weight_packed, layer.vdm_weight_scale_packed, layer.bias, layer.kernel_clip_ratio,
                                      bias_half=layer._bias_half, act=act, residual=residual, gate=gate)
    if act == "gelu_tanh":
        y = F.gelu(y, approximate="tanh")
    out = layer(y)
    if residual is None:
        return out
    return residual + (out if gate is None else out * gate)


class FeedForward(nn.Module):
    def __init__(self, dim: int, ffn_dim: int):
        super().__init__()
        self.up, self.down = nn.Linear(dim, ffn_dim), nn.Linear(ffn_dim, dim)

    fuse_gelu = False  # evaluate the GELU inside the second linear's activation quantizer

    def forward(self, x, residual=None, gate=None) -> torch.Tensor:
        from . import fused_ops

        if isinstance(x, fused_ops.LnInput):
            up = self.up
            y = fused_ops.linear_ln_vdm_w4a4(x, up.vdm_weight_packed, up.vdm_weight_scale_packed, up.bias, up.kernel_clip_ratio,
                                             bias_half=up._bias_half)
        else:
            y = self.up(x)
        if self.fuse_gelu:
            return _project_and_update(self.down, y, "gelu_tanh", residual, gate)
        return _project_and_update(self.down, F.gelu(y, approximate="tanh"), None, residual, gate)


class Block(nn.Module):
    def __init__(self, a: WanArgs):
        super().__init__()
        self.eps = a.eps
        self.attn1 = Attention(a.dim, a.num_heads, a.eps, cross=False)
        self.attn2 = Attention(a.dim, a.num_heads, a.eps, cross=True)
        self.norm2 = nn.LayerNorm(a.dim, a.eps, elementwise_affine=True)
        self.ffn = FeedForward(a.dim, a.ffn_dim)
        self.scale_shift_table = nn.Parameter(torch.randn(1, 6, a.dim) / a.dim ** 0.5)

    fuse_ln = False  # run the three LayerNorms (+ modulation) inside the following linears' activation quantizers
    fuse_residual = False  # run the three residual updates (x + y * gate) in the preceding linears' GEMM epilogues

    def forward(self, x, context, tproj, freqs, timers=None):
        # tproj: [1, 6, dim] (one timestep for the whole sequence; the reference repeats it per token)
        mod = (self.scale_shift_table.to(tproj.dtype) + tproj).unbind(dim=1)
        shift, scale, gate, c_shift, c_scale, c_gate = (m.unsqueeze(1) for m in mod)
        kernel_mode = getattr(self.ffn.up, "use_vdm_kernel", False) and self.attn1.use_fused_qkv_kernel
        if kernel_mode and (self.fuse_ln or self.fuse_residual):
            from .fused_ops import LnInput

            def ln(x, a, b, mode):
                if self.fuse_ln:
                    return LnInput(x, a, b, self.eps, mode)
                if mode == "affine":
                    return fp32_layer_norm(x, a, b, self.eps)
                return fp32_layer_norm(x, None, None, self.eps) * (1 + a) + b

            if self.fuse_residual:
                x = self.attn1(ln(x, scale, shift, "modulate"), None, freqs, timers, residual=x, gate=gate)
                x = self.attn2(ln(x, self.norm2.weight, self.norm2.bias, "affine"), context, None, timers, residual=x)
                return self.ffn(ln(x, c_scale, c_shift, "modulate"), residual=x, gate=c_gate)
            x = x + self.attn1(ln(x, scale, shift, "modulate"), None, freqs, timers) * gate
            x = x + self.attn2(ln(x, self.norm2.weight, self.norm2.bias, "affine"), context, None, timers)
            return x + self.ffn(ln(x, c_scale, c_shift, "modulate")) * c_gate
        h = fp32_layer_norm(x, None, None, self.eps) * (1 + scale) + shift
        x = x + self.attn1(h, None, freqs, timers) * gate
        h = fp32_layer_norm(x, self.norm2.weight, self.norm2.bias, self.eps)
        x = x + self.attn2(h, context, None, timers)
        h = fp32_layer_norm(x, None, None, self.eps) * (1 + c_scale) + c_shift
        return x + self.ffn(h) * c_gate


class WanDiT(nn.Module):
    def __init__(self, a: WanArgs):
        super().__init__()
        self.args = a
        p = a.patch_size
        self.patch_embedding_mlp = nn.Linear(a.in_channels * p[0] * p[1] * p[2], a.dim)
        self.time_embedder = nn.Sequential(nn.Linear(a.freq_dim, a.dim), nn.SiLU(), nn.Linear(a.dim, a.dim))
        self.time_proj = nn.Linear(a.dim, 6 * a.dim)
        self.text_embedder = nn.Sequential(nn.Linear(a.text_dim, a.dim), nn.GELU(approximate="tanh"), nn.Linear(a.dim, a.dim))
        self.blocks = nn.ModuleList([Block(a) for _ in range(a.num_layers)])
        self.proj_out = nn.Linear(a.dim, a.in_channels * p[0] * p[1] * p[2])
        self.scale_shift_table = nn.Parameter(torch.randn(1, 2, a.dim) / a.dim ** 0.5)

    def patchify(self, latent: torch.Tensor) -> torch.Tensor:
        """[1, C, F, H, W] -> [1, F*(H/2)*(W/2), C*4], channel-major inside a patch."""
        _, c, f, h, w = latent.shape
        p1, p2, p3 = self.args.patch_size
        x = latent.reshape(1, c, f // p1, p1, h // p2, p2, w // p3, p3)
        return x.permute(0, 2, 4, 6, 1, 3, 5, 7).reshape(1, (f // p1) * (h // p2) * (w // p3), c * p1 * p2 * p3)

    def unpatchify(self, tokens: torch.Tensor, f: int, h: int, w: int) -> torch.Tensor:
        """[1, L, 4*C] -> [1, C, F, H, W]: the head's output of a token is patch-position major, channel minor
        ('1 l (n c) -> 1 (l n) c' with n = 4, modules/model.py:353), unlike the channel-major input patches."""
        p1, p2, p3 = self.args.patch_size
        c = self.args.in_channels
        x = tokens.reshape(1, f // p1, h // p2, w // p3, p1, p2, p3, c)
        return x.permute(0, 7, 1, 4, 2, 5, 3, 6).reshape(1, c, f, h, w)

    # reuse_context: embed each context tensor once (the prompt's cond / uncond embeddings are the same tensors in
    # every denoise step), keep the blocks' cross-attention K/V per embedded context, and quantize a context that
    # does have to be projected once per forward for all blocks.  Outputs are bit-identical either way.
    reuse_context = False

    def _embedded_context(self, context: torch.Tensor):
        if not self.reuse_context:
            return self.text_embedder(context)
        cache = self.__dict__.setdefault("_context_cache", {})
        ctx = _weak_lookup(cache, context)
        if ctx is None:
            ctx = SharedContext(self.text_embedder(context))
            _weak_store(cache, context, ctx)
        return ctx

    def forward(self, latent: torch.Tensor, timestep: torch.Tensor, context: torch.Tensor, timers=None) -> torch.Tensor:
        """latent [1, C, F, H, W] fp16, timestep [1], context [1, 512, text_dim] -> noise prediction like latent."""
        a = self.args
        _, _, f, h, w = latent.shape
        freqs = rope_frequencies(a.head_dim, f // a.patch_size[0], h // a.patch_size[1], w // a.patch_size[2], latent.device)
        x = self.patch_embedding_mlp(self.patchify(latent))
        temb = self.time_embedder(timestep_embedding(a.freq_dim, timestep).to(x.dtype))
        tproj = self.time_proj(F.silu(temb)).unflatten(1, (6, -1))
        ctx = self._embedded_context(context)
        for blk in self.blocks:
            x = blk(x, ctx, tproj, freqs, timers)
        shift, scale = (self.scale_shift_table.to(temb.dtype) + temb[:, None, :]).unbind(dim=1)
        x = fp32_layer_norm(x, None, None, a.eps) * (1 + scale.unsqueeze(1)) + shift.unsqueeze(1)
        return self.unpatchify(self.proj_out(x), f, h, w)


# ------------------------------------------------------------------ building

def swap_block_linears(model: WanDiT) -> int:
    """Every nn.Linear under ``model.blocks`` becomes a QuantLinear, as
    quant_module_refactor does (scripts/eval_quant_vdm_single.py:149-184)."""
    qp = {"w": {"bit": 4, "sym": True, "granularity": "per_channel"}, "act": {"bit": 4, "sym": True}}
    n = 0

    def walk(mod: nn.Module) -> None:
        nonlocal n
        for name, child in list(mod.named_children()):
            if isinstance(child, nn.Linear):
                setattr(mod, name, QuantLinear(child, {"w": "lsq", "act": "dynamic"}, qp))
                n += 1
            else:
                walk(child)

    walk(model.blocks)
    return n


def synthetic_packed_checkpoint(model: WanDiT, seed: int = 0, device="cpu") -> dict:
    """A ``vdm_w4a4_packed_v1`` checkpoint with random contents for ``model``
    (already swapped): non-quantized parameters ~ N(0, 0.02) (biases 0, norm
    weights 1) as the reference's init_weights; packed weights are uniform
    random nibbles -- any byte pattern is a valid v1 weight buffer --, channel
    scales ~ U(1e-3, 1e-2) replicated per k-group, biases ~ N(0, 0.02)."""
    g = torch.Generator(device=device).manual_seed(seed)
    sd: Dict[str, torch.Tensor] = {}
    quant = {name for name, m in model.named_modules() if isinstance(m, QuantLinear)}
    for key, p in model.state_dict().items():
        if ".wquantizer." in key or ".aquantizer." in key:
            continue
        owner = key.rsplit(".", 1)[0]
        if owner in quant and key.endswith(".weight"):
            continue
        shape = tuple(p.shape)
        if key.endswith("norm_q.weight") or key.endswith("norm_k.weight") or key.endswith("norm2.weight"):
            t = torch.ones(shape, device=device)
        elif key.endswith(".bias") and owner not in quant:
            t = torch.zeros(shape, device=device)
        else:
            t = 0.02 * torch.randn(shape, generator=g, device=device)
        sd[key] = t.half()
    for name in quant:
        m = model.get_submodule(name)
        n, k = m.out_features, m.in_features
        sd[f"{name}.vdm_weight_packed"] = torch.randint(0, 256, (n, k // 2), generator=g, device=device, dtype=torch.uint8)
        scale = (1e-3 + 9e-3 * torch.rand(n, generator=g, device=device)).half()
        sd[f"{name}.vdm_weight_scale"] = scale
        # the GEMM reads k-group 0 of the packed scales; within a 128-row block the v1 order is a
        # permutation of the rows, so the replicated buffer is built with the library's own packer
        sd[f"{name}.vdm_weight_scale_packed"] = _pack_scales_v1(scale, k)
    return {"format": pc.PACKED_CHECKPOINT_FORMAT, "metadata": {"synthetic": True, "seed": seed}, "model": sd}


def _pack_scales_v1(scale: torch.Tensor, k: int) -> torch.Tensor:
    from . import _lib

    if not scale.is_cuda:
        raise RuntimeError("synthetic checkpoints are generated on the GPU (the v1 scale packer is a device kernel)")
    lib = _lib.load()
    out = torch.empty((scale.numel(), k // 64), dtype=torch.float16, device=scale.device)
    _lib.check(lib.vdmq_wscale_plain_to_v1(scale.data_ptr(), out.data_ptr(), scale.numel(), k,
                                           torch.cuda.current_stream(scale.device).cuda_stream))
    return out


def build_quantized(args: WanArgs, device, seed: int = 0) -> WanDiT:
    """Model on the meta device -> QuantLinear swap -> synthetic packed checkpoint ->
    the packed loader -> fused QKV switches: the fast path of
    scripts/eval_quant_vdm_single.py:222-262 with random weights."""
    with torch.device("meta"):
        model = WanDiT(args)
    swap_block_linears(model)
    ckpt = synthetic_packed_checkpoint(model, seed, device=device)
    missing, unexpected = pc.load_packed_quantized_model(model, ckpt, quant_linear_cls=QuantLinear, dtype=torch.float16,
                                                        device=torch.device(device), require_vdm_kernel=True)
    assert not missing and not unexpected, (missing, unexpected)
    pc.enable_fused_qkv(model, quant_linear_cls=QuantLinear, attention_cls=Attention, use_fused_qkv=True)
    return model.eval()


# ------------------------------------------------------------------ timing

class KernelTimers:
    """Event pairs around named regions; totals in ms after ``collect()``."""

    def __init__(self):
        self.pairs: Dict[str, List[Tuple[torch.cuda.Event, torch.cuda.Event]]] = {}
        self._open: Dict[str, torch.cuda.Event] = {}

    def start(self, name: str) -> None:
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        self._open[name] = e

    def stop(self, name: str) -> None:
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        self.pairs.setdefault(name, []).append((self._open.pop(name), e))

    def collect(self) -> Dict[str, float]:
        torch.cuda.synchronize()
        return {k: sum(a.elapsed_time(b) for a, b in v) for k, v in self.pairs.items()}

    def counts(self) -> Dict[str, int]:
        return {k: len(v) for k, v in self.pairs.items()}


class time_w4a4_calls:
    """Context manager: wraps the W4A4 linear entry points so that every W4A4 call is bracketed by events."""

    def __init__(self, timers: KernelTimers):
        self.timers = timers

    def __enter__(self):
        from . import fused_ops
        from .kernels import vdm_w4a4 as k

        timers = self.timers

        def wrap(orig):
            def timed(*a, **kw):
                timers.start("w4a4")
                try:
                    return orig(*a, **kw)
                finally:
                    timers.stop("w4a4")

            return timed

        self._saved = [(k, "linear_vdm_w4a4", k.linear_vdm_w4a4), (k, "linear_vdm_w4a4_prepared", k.linear_vdm_w4a4_prepared),
                       (fused_ops, "linear_fused", fused_ops.linear_fused)]
        for mod, name, orig in self._saved:
            setattr(mod, name, wrap(orig))
        return self

    def __exit__(self, *exc):
        for mod, name, orig in self._saved:
            setattr(mod, name, orig)
        return False


@torch.no_grad()
def denoise(model: WanDiT, latents: torch.Tensor, cond: torch.Tensor, uncond: torch.Tensor, timesteps: List[float],
            guidance_scale: float = 5.0, guidance_scale_2: float = 1.0, boundary_ratio: Optional[float] = 0.4,
            timers: Optional[KernelTimers] = None) -> Tuple[torch.Tensor, int]:
    """Denoise-loop control flow of the reference pipeline; returns (latents, number of forwards)."""
    boundary = None if boundary_ratio is None else boundary_ratio * 1000.0
    forwards = 0
    ts = list(timesteps) + [0.0]
    for i, t in enumerate(timesteps):
        scale = guidance_scale if boundary is None or t >= boundary else guidance_scale_2
        tt = torch.tensor([t], device=latents.device, dtype=torch.float32)
        x = latents.half()
        noise = model(x, tt, cond, timers).float()
        forwards += 1
        if guidance_scale > 1.0 and scale > 1.0:
            noise_u = model(x, tt, uncond, timers).float()
            forwards += 1
            noise = noise_u + scale * (noise - noise_u)
        latents = latents + (ts[i + 1] - t) / 1000.0 * noise  # Euler step of the flow ODE
    return latents, forwards


def unipc_timesteps(num_steps: int, shift: float = 3.0, num_train: int = 1000) -> List[float]:
    """Timesteps of FlowUniPCMultistepScheduler.set_timesteps (schedulers/flow_match_unipc.py:155-201):
    sigmas = linspace(sigma_max, sigma_min, n+1)[:-1] with sigma_max = 1 - 1/num_train, sigma_min = 0,
    shifted by shift*s/(1+(shift-1)*s), times num_train, truncated to integers.
    Five steps at shift 3 give 999, 922, 817, 666, 428: none is below a boundary of 400."""
    sigma_max = 1.0 - 1.0 / num_train
    out = []
    for i in range(num_steps):
        s = sigma_max * (1.0 - i / num_steps)
        out.append(float(int(shift * s / (1 + (shift - 1) * s) * num_train)))
    return out
