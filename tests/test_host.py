"""CPU-side checks: the C ABI loads and exports what include/vdmq.h declares,
and the host logic that mirrors the reference's Python modules (QuantLinear,
packed checkpoints, fused-QKV dispatch) behaves like the source it restates.
No compute call is made on the library here (there is no GPU)."""
import re
from pathlib import Path

import numpy as np
import pytest
import torch
import torch.nn as nn

ROOT = Path(__file__).resolve().parents[1]


def test_library_exports_every_declared_symbol():
    from dsaquant_amd import _lib

    header = (ROOT / "include" / "vdmq.h").read_text()
    declared = set(re.findall(r"\b(vdmq_[a-z0-9_]+)\s*\(", header))
    declared.discard("vdmq_stream_t")
    assert declared, "no declarations found"
    lib = _lib.load()
    for name in sorted(declared):
        assert hasattr(lib, name), f"libvdmq.so does not export {name}"
    assert declared == set(_lib.SIGNATURES), "ctypes signatures and header disagree"
    # pure host calls
    assert lib.vdmq_version() == _lib.VDMQ_VERSION == 2
    assert lib.vdmq_arch() == b"gfx950"
    assert lib.vdmq_k_padded(64) % 64 == 0 and lib.vdmq_k_padded(64) >= 64
    assert lib.vdmq_k_padded(5120) == 5120
    assert lib.vdmq_workspace_bytes(100, 1536) >= 100 * 768 + 200


def test_abi_rejects_bad_shapes_without_touching_the_gpu():
    from dsaquant_amd import _lib

    lib = _lib.load()
    fake = 4096  # a non-null, 16-byte aligned address; never dereferenced because the checks fail first
    assert lib.vdmq_quantize_act(fake, 4, 96, 96, 1.0, fake, fake, None) == -2
    assert b"K must be" in lib.vdmq_last_error()
    assert lib.vdmq_gemm_w4a4(fake, fake, fake, fake, None, fake, 0, 4, 64, 128, 64, None) == -2
    assert b"N must be" in lib.vdmq_last_error()
    assert lib.vdmq_gemm_w4a4(None, fake, fake, fake, None, fake, 0, 4, 128, 128, 128, None) == -1
    assert lib.vdmq_gemm_w4a4(fake, fake, fake + 4, fake, None, fake, 0, 4, 128, 128, 128, None) == -1
    assert b"aligned" in lib.vdmq_last_error()
    assert lib.vdmq_gemm_w4a4(fake, fake, fake, fake, None, fake, 7, 4, 128, 128, 128, None) == -1
    assert lib.vdmq_linear_w4a4(fake, 4, 128, 128, 1.0, fake, fake, None, fake, 0, 128, 128, fake, 16, None) == -4
    assert lib.vdmq_act_v1_to_native(fake, fake, 100, 128, fake, fake, None) == -2
    # the entry point with the built-in workspace refuses what does not fit it, before it looks for a device
    assert lib.vdmq_linear_w4a4_noalloc(fake, 75600, 5120, 5120, 1.0, fake, fake, None, fake, 0, 128, 128, None) == -4
    assert b"scratch" in lib.vdmq_last_error()
    assert lib.vdmq_quantize_act(fake, 0, 128, 128, 1.0, fake, fake, None) == 0  # empty input is fine
    with pytest.raises(_lib.VdmqError):
        _lib.check(-2)


def test_kernel_wrapper_is_unavailable_without_a_gpu_and_never_falls_back():
    from dsaquant_amd.kernels import vdm_w4a4 as v

    if torch.cuda.is_available():
        pytest.skip("GPU present")
    assert v.is_available() is False
    assert v.load_error() is not None
    with pytest.raises(BaseException):
        v.linear_vdm_w4a4(torch.zeros(4, 128), torch.zeros(128, 64, dtype=torch.uint8), torch.zeros(128, 2, dtype=torch.float16))
    assert (v.BLOCK_M, v.BLOCK_N, v.WARP_K) == (256, 128, 64)
    assert v.build_config()["arch_list"] == "gfx950"


def _qparams():
    return {"w": {"bit": 4, "sym": True, "granularity": "per_channel", "group_size": -1, "round_zero": True, "use_grad_scaling": True, "cali": "mse"},
            "act": {"bit": 4, "sym": True}}


def _make_ql(i=64, o=128, bias=True):
    from dsaquant_amd.quantization.quant_linear import QuantLinear

    return QuantLinear(nn.Linear(i, o, bias=bias), {"w": "lsq", "act": "dynamic"}, _qparams())


def test_quantlinear_attributes_and_fake_quant_path():
    torch.manual_seed(1)
    ql = _make_ql()
    for name, val in dict(use_wq=False, use_aq=False, use_hadamard=False, use_timestep_scaling=False, use_kernel=False,
                          use_kernel_fused=False, use_vdm_kernel=False, kernel_clip_ratio=0.95, _bias_half=None, in_features=64,
                          out_features=128).items():
        assert getattr(ql, name) == val
    x = torch.randn(9, 64)
    y_fp = ql(x)
    assert torch.allclose(y_fp, torch.nn.functional.linear(x, ql.weight, ql.bias))
    ql.set_quant_state(use_wq=True, use_aq=True)
    y = ql(x)
    # closed form of the fake-quant path: symmetric int4, scale = absmax/7 clamped at 1e-5, per row
    ws = ql.weight.detach().abs().amax(dim=1, keepdim=True).clamp(min=1e-5) / 7
    wq = torch.clamp(torch.round(ql.weight.detach() / ws), -8, 7) * ws
    xs = x.abs().amax(dim=1, keepdim=True).clamp(min=1e-5) / 7
    xq = torch.clamp(torch.round(x / xs), -8, 7) * xs
    assert torch.allclose(y, torch.nn.functional.linear(xq, wq, ql.bias), atol=1e-6)
    assert torch.equal(ql.wquantizer.scale, ws)
    # the activation scale is frozen after the first call (quant_linear.py:77-78)
    y2 = ql(x * 100)
    xq2 = torch.clamp(torch.round(x * 100 / xs), -8, 7) * xs
    assert torch.allclose(y2, torch.nn.functional.linear(xq2, wq, ql.bias), atol=1e-6)
    assert "use_vdm_kernel=False" in ql.extra_repr()
    with pytest.raises(NotImplementedError):
        ql.set_hadamard(True)
    keys = set(ql.state_dict())
    assert {"weight", "bias", "wquantizer.scale", "aquantizer.scale"} <= keys


def test_uniform_quantizer_asymmetric_and_granularities():
    from dsaquant_amd.quantization.quant_linear import UniformQuantizer

    x = torch.tensor([[0.0, 1.0, 2.0, 3.0], [-1.0, 0.0, 1.0, 15.0]])
    q = UniformQuantizer(bit=4, sym=False)
    y = q(x)
    assert torch.allclose(y[0], x[0], atol=1e-6)  # 0..3 on a 16-level grid of step 0.2
    assert (q.P, q.N) == (15, 0) and q.zero_point is not None
    for gran, rows in (("per_tensor", 1), ("per_channel", 2), ("per_token", 2)):
        u = UniformQuantizer(granularity=gran)
        u(x)
        assert u.scale.shape[0] == rows
    with pytest.raises(ValueError):
        UniformQuantizer(granularity="nope")(x)
    g = UniformQuantizer(granularity="per_group", group_size=2)
    g(x)
    assert g.scale.shape[0] == 4


def test_enable_kernel_mode_fails_loudly_without_the_library_or_gpu():
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    ql = _make_ql()
    ql.wquantizer(ql.weight.detach())
    with pytest.raises(AssertionError, match="not compiled/available"):
        ql.enable_vdm_kernel_mode()
    assert ql.use_vdm_kernel is False and ql.weight is not None


class _Attn(nn.Module):
    def __init__(self, dim=128, cross=False):
        super().__init__()
        self.to_q, self.to_k, self.to_v = _make_ql(dim, dim), _make_ql(dim, dim), _make_ql(dim, dim)
        self.cross_attention_dim_head = 64 if cross else None
        self.fused_projections = False


class _Toy(nn.Module):
    def __init__(self):
        super().__init__()
        self.pre = nn.Linear(8, 128)
        self.blocks = nn.ModuleList([_Attn(), _Attn(cross=True)])


def _synthetic_packed_ckpt(model, legacy=False):
    from dsaquant_amd.checkpoints import packed_checkpoint as pc
    from dsaquant_amd.quantization.quant_linear import QuantLinear

    sd = {}
    for k, v in model.state_dict().items():
        if ".wquantizer." in k or ".aquantizer." in k:
            continue
        sd[k] = v.detach().clone()
    sfx = pc._LEGACY_BUFFER_SUFFIXES if legacy else pc.VDM_BUFFER_SUFFIXES
    for name, m in model.named_modules():
        if isinstance(m, QuantLinear):
            n, k = m.out_features, m.in_features
            del sd[f"{name}.weight"]
            sd[f"{name}.{sfx[0]}"] = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8)
            sd[f"{name}.{sfx[1]}"] = torch.rand(n, k // 64).half()
            sd[f"{name}.{sfx[2]}"] = torch.rand(n).half()
    fmt = pc._LEGACY_PACKED_CHECKPOINT_FORMAT if legacy else pc.PACKED_CHECKPOINT_FORMAT
    return {"format": fmt, "metadata": {"note": "synthetic"}, "model": sd}


@pytest.mark.parametrize("legacy", [False, True])
def test_packed_checkpoint_loader_contract(legacy, tmp_path):
    from dsaquant_amd.checkpoints import packed_checkpoint as pc
    from dsaquant_amd.quantization.quant_linear import QuantLinear

    torch.manual_seed(0)
    src = _Toy()
    ckpt = _synthetic_packed_ckpt(src, legacy)
    assert pc.is_packed_checkpoint(ckpt) and not pc.is_packed_checkpoint({"model": {}}) and not pc.is_packed_checkpoint([1])
    # through a file, with the safe loader
    path = str(tmp_path / "packed.pt")
    torch.save(ckpt, path)
    loaded = pc.load_quant_checkpoint(path, dcp_loader=lambda p: pytest.fail("dcp loader must not be used for .pt"))
    assert pc.load_quant_checkpoint("some_dir", dcp_loader=lambda p: {"dcp": p}) == {"dcp": "some_dir"}

    model = _Toy()
    missing, unexpected = pc.load_packed_quantized_model(model, loaded, quant_linear_cls=QuantLinear, dtype=torch.float16,
                                                        device=torch.device("cpu"), require_vdm_kernel=False)
    assert missing == [] and unexpected == []
    n = 0
    for name, m in model.named_modules():
        if isinstance(m, QuantLinear):
            n += 1
            assert m.use_vdm_kernel and not m.use_kernel and m.weight is None and m.wquantizer is None and m.aquantizer is None
            assert m.use_wq and m.use_aq
            assert m.vdm_weight_packed.dtype == torch.uint8 and m.vdm_weight_scale_packed.dtype == torch.float16
            assert m._bias_half.dtype == torch.float16 and torch.equal(m._bias_half, m.bias.half())
            key = f"{name}.{(pc._LEGACY_BUFFER_SUFFIXES if legacy else pc.VDM_BUFFER_SUFFIXES)[0]}"
            assert torch.equal(m.vdm_weight_packed, ckpt["model"][key])
    assert n == 6
    assert model.pre.weight.dtype == torch.float16 and torch.equal(model.pre.weight, src.pre.weight.half())

    # exporter: what goes back to disk
    sd = pc.packed_state_dict_from_model(model)
    assert not any(".wquantizer." in k or ".aquantizer." in k or k.endswith("._bias_half") or k.endswith("to_q.weight") for k in sd)
    assert sd["blocks.0.to_q.vdm_weight_packed"].dtype == torch.uint8
    out = str(tmp_path / "again.pt")
    pc.save_packed_checkpoint(model, out, metadata={"a": 1})
    again = torch.load(out, weights_only=True)
    assert again["format"] == pc.PACKED_CHECKPOINT_FORMAT and again["metadata"] == {"a": 1}
    assert set(again["model"]) == set(sd)

    pc.enable_fused_qkv(model, quant_linear_cls=QuantLinear, attention_cls=_Attn, use_fused_qkv=True)
    assert all(b.use_fused_qkv_kernel and b.qkv_kernel_backend == "vdm" for b in model.blocks)


def test_packed_checkpoint_loader_errors():
    from dsaquant_amd.checkpoints import packed_checkpoint as pc
    from dsaquant_amd.quantization.quant_linear import QuantLinear

    kw = dict(quant_linear_cls=QuantLinear, dtype=torch.float16, device=torch.device("cpu"), require_vdm_kernel=False)
    with pytest.raises(ValueError, match="Unsupported checkpoint format"):
        pc.load_packed_quantized_model(_Toy(), {"format": "other", "model": {}}, **kw)
    ckpt = _synthetic_packed_ckpt(_Toy())
    del ckpt["model"]["blocks.1.to_k.vdm_weight_scale"]
    with pytest.raises(KeyError, match="missing 1 VDM buffers"):
        pc.load_packed_quantized_model(_Toy(), ckpt, **kw)
    plain = nn.Sequential(nn.Linear(4, 4))
    with pytest.raises(RuntimeError, match="No QuantLinear"):
        pc.load_packed_quantized_model(plain, {"format": pc.PACKED_CHECKPOINT_FORMAT, "model": plain.state_dict()}, **kw)
    if not torch.cuda.is_available():
        with pytest.raises(AssertionError):
            pc.load_packed_quantized_model(_Toy(), _synthetic_packed_ckpt(_Toy()), quant_linear_cls=QuantLinear,
                                           dtype=torch.float16, device=torch.device("cpu"))


def test_fused_qkv_dispatch_falls_through_to_separate_projections_on_cpu():
    from dsaquant_amd.fused_qkv import get_qkv_projections

    torch.manual_seed(3)
    attn = _Attn()
    x = torch.randn(2, 5, 128)
    q, k, v = get_qkv_projections(attn, x, None)
    assert torch.equal(q, attn.to_q(x)) and torch.equal(k, attn.to_k(x)) and torch.equal(v, attn.to_v(x))
    enc = torch.randn(2, 3, 128)
    cross = _Attn(cross=True)
    q, k, v = get_qkv_projections(cross, x, enc)
    assert q.shape == (2, 5, 128) and k.shape == (2, 3, 128) and torch.equal(v, cross.to_v(enc))
    # fp fused projections (attention.py:109-116)
    attn.fused_projections = True
    attn.to_qkv = nn.Linear(128, 384)
    q, k, v = get_qkv_projections(attn, x, None)
    assert torch.equal(torch.cat([q, k, v], -1), attn.to_qkv(x))


def test_concatenated_buffers_carry_the_reference_names_and_share_storage():
    """fused_qkv.concatenated on CPU tensors (no kernel involved): `_vdm_qkv_weight_packed` / `_vdm_qkv_weight_scale`
    (`_vdm_kv_*` for cross-attention) are torch.cat of the projections' v1 buffers as attention.py:44-54, 80-88 of the
    reference builds them; the projections' buffers become views of them (state dict unchanged); a replaced buffer
    makes the cache stale and it is rebuilt."""
    from dsaquant_amd.checkpoints import packed_checkpoint as pc
    from dsaquant_amd.fused_qkv import concatenated
    from dsaquant_amd.quantization.quant_linear import QuantLinear

    torch.manual_seed(1)
    model = _Toy()
    pc.load_packed_quantized_model(model, _synthetic_packed_ckpt(_Toy()), quant_linear_cls=QuantLinear, dtype=torch.float16,
                                   device=torch.device("cpu"), require_vdm_kernel=False)
    sd0 = {k: v.clone() for k, v in model.state_dict().items()}
    attn, cross = model.blocks
    w, s = concatenated(attn, ["to_q", "to_k", "to_v"])
    assert w is attn._vdm_qkv_weight_packed and s is attn._vdm_qkv_weight_scale
    assert torch.equal(w, torch.cat([sd0[f"blocks.0.{n}.vdm_weight_packed"] for n in ("to_q", "to_k", "to_v")]))
    assert torch.equal(s, torch.cat([sd0[f"blocks.0.{n}.vdm_weight_scale_packed"] for n in ("to_q", "to_k", "to_v")]))
    assert attn.to_k.vdm_weight_packed.data_ptr() == w[128:].data_ptr() and attn.to_k.vdm_weight_packed.is_contiguous()
    wkv, _ = concatenated(cross, ["to_k", "to_v"])
    assert wkv is cross._vdm_kv_weight_packed and wkv.shape == (256, 64) and not hasattr(cross, "_vdm_qkv_weight_packed")
    assert cross.to_q.vdm_weight_packed.data_ptr() != wkv.data_ptr()
    sd1 = model.state_dict()
    assert set(sd1) == set(sd0) and all(torch.equal(sd1[k], sd0[k]) for k in sd0)
    assert concatenated(attn, ["to_q", "to_k", "to_v"])[0] is w  # cached
    # a buffer replaced behind the cache's back (what model.to(...) or a checkpoint load does)
    new_k = torch.randint(0, 256, (128, 64), dtype=torch.uint8)
    attn.to_k._buffers["vdm_weight_packed"] = new_k.clone()
    w2, _ = concatenated(attn, ["to_q", "to_k", "to_v"])
    assert w2 is not w and torch.equal(w2[128:256], new_k) and torch.equal(w2[:128], sd0["blocks.0.to_q.vdm_weight_packed"])


# ---- the reference's torch floating-point path, from vectors recorded with its own quant_linear.py ----

_QL_FIXTURE = Path(__file__).parent / "golden" / "quantlinear_fp_path.npz"
_QL_QUANTIZERS = {
    "sym_per_channel": dict(bit=4, sym=True),
    "sym_clip": dict(bit=4, sym=True, clip_ratio=0.9),
    "sym_per_token_3d": dict(bit=4, sym=True, granularity="per_token"),
    "sym_per_channel_3d": dict(bit=4, sym=True),
    "sym_per_tensor": dict(bit=8, sym=True, granularity="per_tensor"),
    "sym_per_group": dict(bit=4, sym=True, granularity="per_group", group_size=8),
    "asym_round_zero": dict(bit=4, sym=False),
    "asym_no_round_zero": dict(bit=4, sym=False, round_zero=False),
    "sym_fp16": dict(bit=4, sym=True),
}


def _bits(a: np.ndarray) -> np.ndarray:
    return a.view({2: np.uint16, 4: np.uint32}[a.dtype.itemsize])


@pytest.mark.parametrize("name", sorted(_QL_QUANTIZERS))
def test_uniform_quantizer_reproduces_the_reference_vectors(name):
    """UniformQuantizer on the recorded inputs: scale, zero point and both fake-quantized tensors (the second one
    with the parameters frozen by the first) are the reference's bits -- elementwise IEEE operations only
    (tests/golden/make_quantlinear_fixture.py wrote the vectors from quant_linear.py:6-86)."""
    from dsaquant_amd.quantization.quant_linear import UniformQuantizer

    g = np.load(_QL_FIXTURE)
    q = UniformQuantizer(**_QL_QUANTIZERS[name])
    y = q(torch.from_numpy(g[f"q.{name}.x"]))
    y2 = q(torch.from_numpy(g[f"q.{name}.x2"]))
    assert np.array_equal(_bits(q.scale.numpy()), _bits(g[f"q.{name}.scale"]))
    if f"q.{name}.zero_point" in g.files:
        assert np.array_equal(_bits(q.zero_point.numpy()), _bits(g[f"q.{name}.zero_point"]))
    else:
        assert q.zero_point is None
    assert np.array_equal(_bits(y.numpy()), _bits(g[f"q.{name}.y"]))
    assert np.array_equal(_bits(y2.numpy()), _bits(g[f"q.{name}.y2"]))


@pytest.mark.parametrize("name,bias", [("bias_2d", True), ("nobias_2d", False), ("bias_3d", True)])
def test_quantlinear_fp_path_reproduces_the_reference_vectors(name, bias):
    """QuantLinear.forward without the kernel on the recorded layer and inputs (quant_linear.py:162-178): plain,
    weight-only, weight + activation, and a second input under the activation scale the first one froze.  The
    quantizer scales are exact; the outputs go through F.linear, whose fp32 summation order belongs to the torch
    build, hence 1e-5 of the largest output."""
    from dsaquant_amd.quantization.quant_linear import QuantLinear

    g = np.load(_QL_FIXTURE)
    layer = nn.Linear(40, 24, bias=bias)
    with torch.no_grad():
        layer.weight.copy_(torch.from_numpy(g[f"l.{name}.weight"]))
        if bias:
            layer.bias.copy_(torch.from_numpy(g[f"l.{name}.bias"]))
    m = QuantLinear(layer, {"w": "lsq", "act": "dynamic"}, {"w": {"bit": 4, "sym": True}, "act": {"bit": 4, "sym": True}})
    x, x2 = torch.from_numpy(g[f"l.{name}.x"]), torch.from_numpy(g[f"l.{name}.x2"])
    with torch.no_grad():
        got = {"plain": m(x)}
        m.set_quant_state(True, False)
        got["w_only"] = m(x)
        m.set_quant_state(True, True)
        got["both"] = m(x)
        got["both2"] = m(x2)
    assert np.array_equal(_bits(m.wquantizer.scale.numpy()), _bits(g[f"l.{name}.wscale"]))
    assert np.array_equal(_bits(m.aquantizer.scale.numpy()), _bits(g[f"l.{name}.ascale"]))
    for key, y in got.items():
        want = g[f"l.{name}.{key}"]
        assert y.shape == want.shape
        assert np.abs(y.numpy() - want).max() <= 1e-5 * np.abs(want).max(), key
    assert m.extra_repr() == str(g[f"l.{name}.repr"])


def test_cpu_baseline_restatement_matches_the_reference_vectors():
    """oracle/quantlinear_torch.py (the timed CPU baseline) on the recorded 2-D cases: its scales are the reference's
    bits; with `dynamic=False` (scale frozen by the first call, as the reference does) both outputs agree to the
    F.linear tolerance, and `dynamic=True` differs from the reference only by recomputing the scale per call."""
    from oracle.quantlinear_torch import QuantLinearTorchPath, sym_scale

    g = np.load(_QL_FIXTURE)
    for name, bias in (("bias_2d", True), ("nobias_2d", False)):
        w = torch.from_numpy(g[f"l.{name}.weight"])
        b = torch.from_numpy(g[f"l.{name}.bias"]) if bias else None
        x, x2 = torch.from_numpy(g[f"l.{name}.x"]), torch.from_numpy(g[f"l.{name}.x2"])
        p = QuantLinearTorchPath(w, b, dynamic=False)
        y, y2 = p(x), p(x2)
        assert np.array_equal(_bits(p.wscale.numpy()), _bits(g[f"l.{name}.wscale"]))
        assert np.array_equal(_bits(p.ascale.numpy()), _bits(g[f"l.{name}.ascale"]))
        for got, key in ((y, "both"), (y2, "both2")):
            want = g[f"l.{name}.{key}"]
            assert np.abs(got.numpy() - want).max() <= 1e-5 * np.abs(want).max(), (name, key)
        d = QuantLinearTorchPath(w, b, dynamic=True)
        assert np.abs(d(x).numpy() - g[f"l.{name}.both"]).max() <= 1e-5 * np.abs(g[f"l.{name}.both"]).max()
        d(x2)
        assert np.array_equal(_bits(d.ascale.numpy()), _bits(sym_scale(x2).numpy()))


# ---- a checkpoint written by the reference's own writer, and what its own loader makes of it ----

def _checkpoint_fixture():
    import importlib.util
    import json

    golden = Path(__file__).parent / "golden"
    spec = importlib.util.spec_from_file_location("_make_checkpoint_fixture", golden / "make_checkpoint_fixture.py")
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)  # for build_toy and describe only; its main() is what touches the reference
    return golden, gen, json.loads((golden / "reference_loader_outcome.json").read_text())


@pytest.mark.parametrize("tag", ["v1", "legacy"])
def test_reference_written_checkpoint_loads_as_the_reference_loads_it(tag):
    """tests/golden/reference_written_packed_{v1,legacy}.pt were written by the reference's save_packed_checkpoint
    (packed_checkpoint.py:190-215) from a toy model of its own QuantLinear layers; reference_loader_outcome.json is
    what its load_packed_quantized_model (:52-148) left behind.  This repository's loader on this repository's
    QuantLinear ends in the same state: missing / unexpected keys, every flag of the layers, dropped fp weight and
    quantizers, buffer names, dtypes and shapes of the state dict, and the keys a re-export would write."""
    from dsaquant_amd.checkpoints import packed_checkpoint as pc
    from dsaquant_amd.quantization.quant_linear import QuantLinear

    golden, gen, want = _checkpoint_fixture()
    path = str(golden / f"reference_written_packed_{tag}.pt")
    ckpt = pc.load_quant_checkpoint(path, dcp_loader=None)
    assert pc.is_packed_checkpoint(ckpt) == want["is_packed_checkpoint"][tag] is True
    if tag == "v1":
        assert ckpt["format"] == want["format"] == pc.PACKED_CHECKPOINT_FORMAT and ckpt["metadata"] == want["metadata"]
        assert {k: [str(v.dtype), list(v.shape)] for k, v in ckpt["model"].items()} == want["saved_keys"]
    model = gen.build_toy(QuantLinear, seed=1)
    missing, unexpected = pc.load_packed_quantized_model(model, ckpt, quant_linear_cls=QuantLinear, dtype=torch.float16,
                                                        device=torch.device("cpu"), require_vdm_kernel=False)
    got = gen.describe(model, QuantLinear)
    ref = want["loads"][tag]
    assert list(missing) == ref["missing"] and list(unexpected) == ref["unexpected"]
    assert got["layers"] == ref["layers"]
    assert got["state_dict"] == ref["state_dict"]
    assert {k: [str(v.dtype), list(v.shape)] for k, v in pc.packed_state_dict_from_model(model).items()} == ref["re_export"]
    # the tensors themselves are the file's
    sfx = dict(zip(pc.VDM_BUFFER_SUFFIXES, pc._LEGACY_BUFFER_SUFFIXES if tag == "legacy" else pc.VDM_BUFFER_SUFFIXES))
    for name in ("q1", "q2"):
        for new, stored in sfx.items():
            assert torch.equal(getattr(getattr(model, name), new), ckpt["model"][f"{name}.{stored}"])
    assert torch.equal(model.pre.weight, ckpt["model"]["pre.weight"]) and torch.equal(model.q1.bias, ckpt["model"]["q1.bias"])


def test_writer_writes_what_the_reference_writer_wrote(tmp_path):
    """save_packed_checkpoint on the model loaded from the reference-written file gives a file with the same
    format string and, key for key, the same dtypes, shapes and bytes as the reference's re-export would hold."""
    from dsaquant_amd.checkpoints import packed_checkpoint as pc
    from dsaquant_amd.quantization.quant_linear import QuantLinear

    golden, gen, want = _checkpoint_fixture()
    ckpt = torch.load(str(golden / "reference_written_packed_v1.pt"), map_location="cpu", weights_only=True)
    model = gen.build_toy(QuantLinear, seed=2)
    pc.load_packed_quantized_model(model, ckpt, quant_linear_cls=QuantLinear, dtype=torch.float16, device=torch.device("cpu"),
                                   require_vdm_kernel=False)
    out = str(tmp_path / "rewritten.pt")
    pc.save_packed_checkpoint(model, out, metadata=ckpt["metadata"])
    again = torch.load(out, map_location="cpu", weights_only=True)
    assert again["format"] == want["format"] and again["metadata"] == want["metadata"]
    assert {k: [str(v.dtype), list(v.shape)] for k, v in again["model"].items()} == want["loads"]["v1"]["re_export"]
    for k, v in again["model"].items():
        assert torch.equal(v, ckpt["model"][k]), k


def test_loader_errors_read_as_the_reference_loader_errors():
    from dsaquant_amd.checkpoints import packed_checkpoint as pc
    from dsaquant_amd.quantization.quant_linear import QuantLinear

    golden, gen, want = _checkpoint_fixture()
    ckpt = torch.load(str(golden / "reference_written_packed_v1.pt"), map_location="cpu", weights_only=True)
    kw = dict(quant_linear_cls=QuantLinear, dtype=torch.float16, device=torch.device("cpu"), require_vdm_kernel=False)
    plain = nn.Sequential(nn.Linear(4, 4))
    cases = {
        "missing_buffer": lambda: pc.load_packed_quantized_model(
            gen.build_toy(QuantLinear), dict(ckpt, model={k: v for k, v in ckpt["model"].items() if k != "q2.vdm_weight_scale"}), **kw),
        "other_format": lambda: pc.load_packed_quantized_model(gen.build_toy(QuantLinear), {"format": "other", "model": {}}, **kw),
        "not_a_dict": lambda: pc.load_packed_quantized_model(gen.build_toy(QuantLinear), [1, 2], **kw),
        "no_quant_layers": lambda: pc.load_packed_quantized_model(plain, {"format": pc.PACKED_CHECKPOINT_FORMAT, "model": plain.state_dict()}, **kw),
    }
    assert set(cases) == set(want["errors"])
    for name, fn in cases.items():
        with pytest.raises(Exception) as info:
            fn()
        assert [type(info.value).__name__, str(info.value)] == want["errors"][name], name


def test_cache_keys_work_for_tensors_made_under_inference_mode():
    """Inference tensors keep no version counter (reading ``_version`` raises) although they can be written in place
    under inference mode: the caches that watch for in-place writes must not read the counter on them, and must not
    reuse anything derived from one."""
    from dsaquant_amd import wan_harness
    from dsaquant_amd.kernels import vdm_w4a4 as v

    with torch.inference_mode():
        t = torch.zeros(4)
    with pytest.raises(RuntimeError):
        t._version
    assert v._version_of(t) is None and wan_harness._version_of(t) is None
    cache = {}
    wan_harness._weak_store(cache, t, "kept")
    assert wan_harness._weak_lookup(cache, t) is None
    u = torch.zeros(4)
    wan_harness._weak_store(cache, u, "kept too")
    assert wan_harness._weak_lookup(cache, u) == "kept too"
    u.add_(1)  # an ordinary tensor written in place is a miss
    assert wan_harness._weak_lookup(cache, u) is None


def test_library_says_where_the_fp6_path_pays():
    """vdmq_bf6_pays is a pure function of the sizes (no GPU work): with a small-tile configuration in the GEMM it is
    the row length alone that decides (the quantizer that writes 6-bit blocks is the slower one on short rows)."""
    from dsaquant_amd import _lib

    lib = _lib.load()
    pays = lambda M, N, K: bool(lib.vdmq_bf6_pays(M, N, K))  # noqa: E731
    assert pays(75600, 15360, 5120) and pays(75600, 5120, 13824) and pays(32760, 1536, 1536) and pays(27280, 3072, 14336)
    assert pays(4096, 4608, 1536)            # config 0
    assert pays(512, 10240, 5120)            # the skinny cross-attention K/V case of the 14B model
    assert pays(512, 3072, 1536)             # the same of the 1.3B model
    assert pays(1, 128, 1280) and not pays(1, 128, 1216)
    assert not pays(32768, 5120, 1024) and not pays(257, 128, 64)
    assert not pays(0, 128, 5120) and not pays(-1, 128, 5120)


def test_bf6_tile_order_takes_every_tile_once(tmp_path):
    """The tile order of the bf6 GEMM kernels (regrouped edge super-tiles, round-robin and both kinds of contiguous
    runs) enumerated on the host for every grid up to 72 x 72 tiles and the benchmark shapes: tests/tilemap_check.cpp
    includes the header the kernels and their launcher use."""
    import shutil
    import subprocess
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        pytest.skip("no host C++ compiler")
    root = Path(__file__).resolve().parent.parent
    exe = tmp_path / "tilemap_check"
    subprocess.run([cxx, "-O1", "-std=c++17", "-Wall", "-Werror", "-I", str(root / "dsaquant_amd" / "csrc"),
                    str(root / "tests" / "tilemap_check.cpp"), "-o", str(exe)], check=True)
    res = subprocess.run([str(exe)], stdout=subprocess.PIPE, text=True)
    assert res.returncode == 0 and res.stdout.startswith("ok "), res.stdout


def test_header_is_plain_c_and_a_c_host_links_the_library(tmp_path):
    """include/vdmq.h is what a C or C++ host of the reference's kernels would include: it must compile as C99 with
    every warning an error, and a C program must link libvdmq.so by its declarations alone.  The program calls the
    entry points that need no GPU (sizes, the version, the path rule, a rejected shape and its message)."""
    import shutil
    import subprocess

    from dsaquant_amd import _lib

    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no host C compiler")
    _lib.load()  # built, or this raises
    root = Path(__file__).resolve().parent.parent
    src = tmp_path / "host.c"
    src.write_text(r'''
#include <stdio.h>
#include <string.h>
#include "vdmq.h"
int main(void) {
    vdmq_gemm_launch_info info;
    if (vdmq_version() != VDMQ_VERSION) return 1;
    if (vdmq_k_padded(64) != 256 || vdmq_k_padded(5120) != 5120) return 2;
    if (vdmq_workspace_bytes(0, 64) < 0) return 3;
    if (vdmq_bf6_bytes(32, 128) != 32 * 128 * 3 / 4) return 4;
    if (!vdmq_bf6_pays(75600, 15360, 5120) || vdmq_bf6_pays(75600, 15360, 64)) return 5;
    if (vdmq_gemm_w4a4(NULL, NULL, NULL, NULL, NULL, NULL, VDMQ_OUT_F16, 16, 100, 64, 100, NULL) == VDMQ_OK) return 6; /* N % 128 */
    if (strlen(vdmq_last_error()) == 0) return 7;
    if (vdmq_last_gemm_launch(&info) == VDMQ_OK) return 8; /* nothing was launched */
    printf("ok %d\n", vdmq_version());
    return 0;
}
''')
    exe = tmp_path / "host"
    lib_dir = _lib.LIB_PATH.parent
    subprocess.run([cc, "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", str(root / "include"), str(src), "-o", str(exe),
                    "-L", str(lib_dir), "-lvdmq", f"-Wl,-rpath,{lib_dir}", "-L/opt/rocm/lib", "-Wl,-rpath,/opt/rocm/lib"], check=True)
    res = subprocess.run([str(exe)], stdout=subprocess.PIPE, text=True)
    assert res.returncode == 0 and res.stdout.startswith("ok "), (res.returncode, res.stdout)
