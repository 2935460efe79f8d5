"""The drop-in surface beyond single calls: what the fused-QKV dispatch leaves on an attention module, which tensors
it returns, the weights kept in one form only (v1 storage released and rebuilt), forms made lazily on one stream and
used on another, and packed buffers that are inference tensors."""
from dataclasses import replace

import numpy as np
import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _small_model(seed=3):
    from dsaquant_amd import wan_harness as W

    args = replace(W.WAN21_1P3B, num_layers=1, num_heads=2, ffn_dim=512, text_dim=128)  # dim 256, head dim 128
    return W, args, W.build_quantized(args, DEV, seed=seed)


def test_fused_qkv_leaves_the_reference_object_graph():
    """get_qkv_projections on a module in fused kernel mode: the concatenated v1 buffers and bias hang on the module
    under the reference's names (attention.py:44-66, 80-98) with the values torch.cat gives, the three results are views
    of ONE [tokens, 3 * dim] tensor (vdm_w4a4.py:297-298), bit-equal to three separate projections; the contiguous
    outputs the harness uses are an opt-in with the same bits."""
    from dsaquant_amd.fused_qkv import get_qkv_projections

    W, args, model = _small_model()
    attn, cross = model.blocks[0].attn1, model.blocks[0].attn2
    parts = [(getattr(attn, n).vdm_weight_packed.clone(), getattr(attn, n).vdm_weight_scale_packed.clone()) for n in ("to_q", "to_k", "to_v")]
    assert torch.equal(attn._vdm_qkv_weight_packed, torch.cat([p[0] for p in parts]))
    assert torch.equal(attn._vdm_qkv_weight_scale, torch.cat([p[1] for p in parts]))
    assert torch.equal(cross._vdm_kv_weight_packed, torch.cat([cross.to_k.vdm_weight_packed, cross.to_v.vdm_weight_packed]))
    assert torch.equal(cross._vdm_kv_weight_scale, torch.cat([cross.to_k.vdm_weight_scale_packed, cross.to_v.vdm_weight_scale_packed]))
    assert not hasattr(cross, "_vdm_qkv_weight_packed") and not hasattr(attn, "_vdm_kv_weight_packed")
    # one copy of the weights: the projections' buffers are views of the concatenation, and still what state_dict() returns
    sd = model.state_dict()
    assert torch.equal(sd["blocks.0.attn1.to_k.vdm_weight_packed"], parts[1][0])
    assert attn.to_v.vdm_weight_packed.untyped_storage().data_ptr() == attn._vdm_qkv_weight_packed.untyped_storage().data_ptr()

    g = torch.Generator(device=DEV).manual_seed(1)
    x = torch.randn((2, 300, args.dim), generator=g, device=DEV).half()
    ctx = torch.randn((2, 77, args.dim), generator=g, device=DEV).half()
    for module, enc, names in ((attn, None, ("to_q", "to_k", "to_v")), (cross, ctx, ("to_k", "to_v"))):
        module.qkv_contiguous_outputs = False  # what a module that never heard of the switch gets: see the default below
        q, k, v = get_qkv_projections(module, x, enc)
        fused = (q, k, v)[3 - len(names):]
        assert len({t.untyped_storage().data_ptr() for t in fused}) == 1  # views of one tensor
        assert all(t.stride(-2) == len(names) * args.dim and not t.is_contiguous() for t in fused)
        want = [getattr(module, n)(x if (enc is None or n == "to_q") else enc) for n in ("to_q", "to_k", "to_v")]
        assert all(torch.equal(a, b) for a, b in zip((q, k, v), want))
        prefix = "_vdm_qkv" if enc is None else "_vdm_kv"
        assert torch.equal(getattr(module, prefix + "_bias_half"), torch.cat([getattr(module, n)._bias_half for n in names]))
        module.qkv_contiguous_outputs = True
        q2, k2, v2 = get_qkv_projections(module, x, enc)
        assert all(t.is_contiguous() for t in (q2, k2, v2)) and all(torch.equal(a, b) for a, b in zip((q2, k2, v2), want))
    # a module without the switch (the reference's WanAttention has none) gets the views
    del attn.qkv_contiguous_outputs
    assert not any(t.is_contiguous() for t in get_qkv_projections(attn, x, None))


@pytest.mark.parametrize("N,K", [(256, 320), (1536, 1536), (128, 64)])
def test_bf6_to_weight_v1_inverts_the_load_time_relayout(N, K):
    """vdmq_weight_v1_to_bf6 followed by vdmq_bf6_to_weight_v1 gives back every byte of an arbitrary v1 buffer (all
    sixteen nibble values, K with and without a padded k-block), and agrees with the relayout through native rows."""
    from dsaquant_amd import _lib

    lib = _lib.load()
    rng = np.random.default_rng(N + K)
    v1 = _dev(rng.integers(0, 256, (N, K // 2), dtype=np.uint8))
    s = torch.cuda.current_stream().cuda_stream
    blocks = torch.full((int(lib.vdmq_bf6_bytes(N, K)),), 0xAB, dtype=torch.uint8, device=DEV)
    back = torch.full_like(v1, 0xCD)
    _lib.check(lib.vdmq_weight_v1_to_bf6(v1.data_ptr(), blocks.data_ptr(), N, K, s))
    _lib.check(lib.vdmq_bf6_to_weight_v1(blocks.data_ptr(), back.data_ptr(), N, K, s))
    torch.cuda.synchronize()
    assert torch.equal(back, v1)
    # the oracle's view of the same buffer: unpack the v1 bytes on the CPU, pack them again
    q = O.np_unpack_wgt_v1(v1.cpu().numpy(), N, K)
    assert np.array_equal(O.np_pack_wgt_v1(q), back.cpu().numpy())
    assert lib.vdmq_bf6_to_weight_v1(blocks.data_ptr(), back.data_ptr(), N + 1, K, None) == -2


@pytest.mark.parametrize("path", ["bf6", "int8"])
def test_v1_storage_released_and_rebuilt(path):
    """A prepared weight can stand in for its v1 buffer: release_v1 frees the buffer's memory (same tensor object, shape
    and device), calls keep giving the same bits, and the bytes come back exactly -- on demand, and before state_dict()."""
    from dsaquant_amd.kernels import vdm_w4a4 as v

    M, K, N = 300, 1536, 1536
    x, qw, ws, bias = O.synth_linear(M, K, N, seed=8)
    q, s, b, xt = _dev(O.np_pack_wgt_v1(qw)), _dev(O.np_pack_wscales_v1(ws, K)), _dev(bias), _dev(x)
    keep = q.clone()
    old = v.matrix_path()
    v.set_matrix_path(path)
    try:
        y0 = v.linear_vdm_w4a4(xt, q, s, b, clip_ratio=0.95)
        pw = q.__dict__["_vdmq_prepared"][0]
        assert (pw.bf6 is not None) == (path == "bf6") and (pw.native is not None) == (path == "int8")
        assert pw.release_v1() == N * K // 2 and q.untyped_storage().nbytes() == 0 and q.shape == (N, K // 2) and q.is_cuda
        assert pw.release_v1() == 0  # nothing left to free
        y1 = v.linear_vdm_w4a4(xt, q, s, b, clip_ratio=0.95)
        assert torch.equal(y0, y1)
        v.ensure_v1(q)
        torch.cuda.synchronize()
        assert q.untyped_storage().nbytes() == N * K // 2 and torch.equal(q, keep)
        v.ensure_v1(q)  # a no-op now
        # dropping the prepared forms of a released buffer brings the bytes back first
        pw.release_v1()
        v.release_prepared(q, concatenations=True)
        assert torch.equal(q, keep) and not q.__dict__["_vdmq_prepared"]
    finally:
        v.set_matrix_path(old)


def test_model_runs_and_exports_with_v1_storage_released():
    """release_v1_storage over a loaded model (also through the loader's release_v1 option): the forward is unchanged,
    state_dict() and the checkpoint writer return every packed byte, the memory is gone in between."""
    from dsaquant_amd import wan_harness as W
    from dsaquant_amd.checkpoints import packed_checkpoint as pc
    from dsaquant_amd.kernels import vdm_w4a4 as v

    W_, args, model = _small_model(seed=5)
    g = torch.Generator(device=DEV).manual_seed(0)
    latent = torch.randn((1, 16, 3, 8, 12), generator=g, device=DEV).half()
    ctx = torch.randn((1, 64, args.text_dim), generator=g, device=DEV).half()
    t = torch.tensor([500.0], device=DEV)
    with torch.no_grad():
        y0 = model(latent, t, ctx)
    sd0 = {k: val.clone() for k, val in model.state_dict().items() if k.endswith("vdm_weight_packed")}
    total = sum(val.numel() for val in sd0.values())
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    freed = v.release_v1_storage(model)
    assert freed == total and torch.cuda.memory_allocated() == before - total
    assert v.release_v1_storage(model) == 0
    with torch.no_grad():
        y1 = model(latent, t, ctx)
    assert torch.equal(y0, y1)
    sd1 = pc.packed_state_dict_from_model(model)  # goes through state_dict(): the hook restores first
    assert all(torch.equal(sd1[k], val.cpu()) for k, val in sd0.items())
    assert v.release_v1_storage(model) == total  # and may be released again
    v.restore_v1_storage(model)
    assert all(torch.equal(model.state_dict()[k], val) for k, val in sd0.items())

    # the loader's option, followed by the fused-QKV switch (which concatenates the released buffers)
    with torch.device("meta"):
        lean = W.WanDiT(args)
    W.swap_block_linears(lean)
    ckpt = W.synthetic_packed_checkpoint(lean, 5, device=DEV)
    pc.load_packed_quantized_model(lean, ckpt, quant_linear_cls=W.QuantLinear, dtype=torch.float16, device=torch.device(DEV), release_v1=True)
    assert all(m.vdm_weight_packed.untyped_storage().nbytes() == 0 for m in lean.modules() if isinstance(m, W.QuantLinear))
    pc.enable_fused_qkv(lean, quant_linear_cls=W.QuantLinear, attention_cls=W.Attention, use_fused_qkv=True)
    assert all(m.vdm_weight_packed.untyped_storage().nbytes() == 0 for m in lean.modules() if isinstance(m, W.QuantLinear))
    with torch.no_grad():
        y2 = lean.eval()(latent, t, ctx)
    assert torch.equal(y0, y2)
    assert all(torch.equal(lean.state_dict()[k], val) for k, val in sd0.items())


def test_lazily_prepared_weight_is_ordered_across_streams():
    """A weight relaid inside its first call is relaid on that call's stream; a call on another stream right after has
    to be ordered behind the relayout (an event recorded behind it, waited for once per stream)."""
    from dsaquant_amd.kernels import vdm_w4a4 as v

    M, K, N = 2000, 3072, 3072
    x, qw, ws, bias = O.synth_linear(M, K, N, seed=12)
    q, s, b, xt = _dev(O.np_pack_wgt_v1(qw)), _dev(O.np_pack_wscales_v1(ws, K)), _dev(bias), _dev(x)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    with torch.cuda.stream(s1):
        y1 = v.linear_vdm_w4a4(xt, q, s, b, clip_ratio=1.0)
    with torch.cuda.stream(s2):
        y2 = v.linear_vdm_w4a4(xt, q, s, b, clip_ratio=1.0)
    torch.cuda.synchronize()
    pw = q.__dict__["_vdmq_prepared"][0]
    form = "bf6" if pw.bf6 is not None else "native"
    assert pw._ready[form][1] == s1.cuda_stream and s2.cuda_stream in pw._ready[form][2] and s2.cuda_stream in pw._ready["wscale"][2]
    rows = np.r_[0:16, M - 16:M]
    want = O.np_linear(x[rows], qw, ws, bias, 1.0)[0]
    for y in (y1, y2):
        assert np.array_equal(y[torch.from_numpy(rows).to(DEV)].cpu().numpy().view(np.uint16), want.view(np.uint16))
    assert torch.equal(y1, y2)


def test_forms_kept_on_inference_tensors_are_not_trusted_at_prepare_time():
    """Buffers made under torch.inference_mode() count no versions, so an in-place write is invisible to the form kept
    with them; prepare_weight (what the loader and enable_vdm_kernel_mode run) makes the form anew."""
    from dsaquant_amd.kernels import vdm_w4a4 as v

    M, K, N = 64, 256, 128
    x, qw_a, ws, bias = O.synth_linear(M, K, N, seed=1)
    qw_b = O.synth_linear(M, K, N, seed=2)[1]
    with torch.inference_mode():
        q, s = _dev(O.np_pack_wgt_v1(qw_a)), _dev(O.np_pack_wscales_v1(ws, K))
        assert q.is_inference()
        v.prepare_weight(q, s)
        ya = v.linear_vdm_w4a4(_dev(x), q, s, _dev(bias), clip_ratio=1.0)
        q.copy_(_dev(O.np_pack_wgt_v1(qw_b)))
        v.prepare_weight(q, s)
        yb = v.linear_vdm_w4a4(_dev(x), q, s, _dev(bias), clip_ratio=1.0)
    assert np.array_equal(ya.cpu().numpy().view(np.uint16), O.np_linear(x, qw_a, ws, bias, 1.0)[0].view(np.uint16))
    assert np.array_equal(yb.cpu().numpy().view(np.uint16), O.np_linear(x, qw_b, ws, bias, 1.0)[0].view(np.uint16))


@pytest.mark.parametrize("K,bf6", [(1536, True), (256, False)])
def test_shared_quantized_input_takes_the_path_of_its_row_length(K, bf6):
    """An input quantized once for several linears (fused_ops.QuantizedInput: the cross-attention context) is held in
    the operand form of the matrix path the library picks for its row length, and every linear fed by it gives the
    bits of the linear that quantizes for itself -- and of the oracle."""
    from dsaquant_amd import fused_ops
    from dsaquant_amd.kernels import vdm_w4a4 as v

    assert v.is_available(), v.load_error()
    M = 512
    x = O.synth_linear(M, K, 128, seed=K)[0]
    shared = fused_ops.QuantizedInput(_dev(x), 1.0)
    assert shared.bf6 is bf6 and v.matrix_path() == "auto"
    for N, seed in ((384, 1), (3072, 2)):
        _, qw, ws, bias = O.synth_linear(1, K, N, seed=seed)
        qv1, sv1, b = _dev(O.np_pack_wgt_v1(qw)), _dev(O.np_pack_wscales_v1(ws, K)), _dev(bias)
        got = fused_ops.linear_fused(shared, qv1, sv1, b, 1.0)
        assert torch.equal(got, v.linear_vdm_w4a4(_dev(x), qv1, sv1, b, clip_ratio=1.0))
        want = O.np_linear(x, qw, ws, bias, 1.0)[0]
        assert np.array_equal(got.cpu().numpy().view(np.uint16), want.view(np.uint16))
