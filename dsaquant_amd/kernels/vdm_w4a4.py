"""W4A4 kernel wrapper for MI355X, function-for-function with the reference's
``vdm_infer/kernels/vdm_w4a4.py`` (same names, arguments, shapes, dtypes and
error types), backed by ``libvdmq.so`` through ctypes instead of a JIT-built
CUDA extension.

What differs underneath (not visible through this API):

* activations are quantized in ONE pass (absmax + quantize) into a row-major
  int4 buffer with one fp16 scale per token -- the v1 fragment-ordered ``qact``
  and the K/64-times replicated ``ascales`` only exist when a caller asks for
  them through ``quantize_activation_per_token``;
* the checkpoint's v1 weight buffers are relaid once per (qweight, wscales)
  pair into the row-major form the gfx950 GEMM consumes, and cached for the
  lifetime of the v1 tensor (the reference caches its concatenated QKV buffers
  the same way, attention.py:44-54).

There is no CPU/PyTorch fallback: without the built library or a GPU every
kernel function raises.
"""
from __future__ import annotations

import os
import weakref
from typing import Dict, Optional, Tuple

import torch

from .. import _lib

BLOCK_M = 256  # vdm_w4a4.py:23-25 of the reference
BLOCK_N = 128
WARP_K = 64

_LOAD_ERROR: Optional[BaseException] = None


def build_config() -> dict:
    """Counterpart of vdm_w4a4.py:115-127: where the native code comes from."""
    return {
        "library": str(_lib.LIB_PATH),
        "arch_list": "gfx950",
        "arch_tag": "gfx950",
        "build_dir": str(_lib.CSRC / "_build"),
        "extension_name": "libvdmq",
        "torch_hip": torch.version.hip,
    }


def _load_ext():
    global _LOAD_ERROR
    try:
        lib = _lib.load()
        if not torch.cuda.is_available():
            raise RuntimeError("no HIP device is visible to torch")
        _LOAD_ERROR = None
        return lib
    except BaseException as exc:  # kept for load_error(), like vdm_w4a4.py:165-167
        _LOAD_ERROR = exc
        raise


def is_available() -> bool:
    """Never raises (vdm_w4a4.py:170-175)."""
    try:
        _load_ext()
        return True
    except BaseException:
        return False


def load_error() -> Optional[BaseException]:
    return _LOAD_ERROR


# ----------------------------------------------------------------- helpers

def _stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _require(cond: bool, msg: str) -> None:
    # the reference's TORCH_CHECK failures surface as RuntimeError
    if not cond:
        raise _lib.VdmqError(msg)


def _check_device_tensor(t: torch.Tensor, name: str, dtype: torch.dtype) -> None:
    _require(t.is_cuda, f"{name} must be a CUDA tensor")  # vdm_w4a4_kernel.cu:688-691
    _require(t.is_contiguous(), f"{name} must be contiguous")
    _require(t.dtype == dtype, f"{name} must be {str(dtype).replace('torch.', '')}")


def _as_2d_half_contiguous(x: torch.Tensor) -> Tuple[torch.Tensor, Tuple[int, ...]]:
    orig_shape = tuple(x.shape[:-1])
    return x.reshape(-1, x.shape[-1]).half().contiguous(), orig_shape


def _check_packed_weight(qweight: torch.Tensor, wscales: torch.Tensor, K: int) -> None:
    # same conditions, order and exception type as vdm_w4a4.py:198-206
    if K % WARP_K != 0:
        raise ValueError(f"K={K} must be a multiple of {WARP_K}")
    if qweight.shape[0] % BLOCK_N != 0:
        raise ValueError(f"N={qweight.shape[0]} must be a multiple of {BLOCK_N}")
    if qweight.shape[1] != K // 2:
        raise ValueError("qweight shape must be [N, K/2]")
    if wscales.shape != (qweight.shape[0], K // WARP_K):
        raise ValueError("wscales shape must be [N, K/64]")


def _check_linear_shapes(x_2d: torch.Tensor, qweight: torch.Tensor, wscales: torch.Tensor) -> None:
    _check_packed_weight(qweight, wscales, x_2d.shape[1])


def k_padded(K: int) -> int:
    return int(_lib.load().vdmq_k_padded(K))


# ------------------------------------------------- the weights in the form the kernels stream
# A checkpoint's v1 buffers stay what the module holds (they are the state-dict contract).  The kernels want the
# same integers either as native int4 rows (int8 matrix path) or as bf6 blocks (bf6 path), plus one fp16 scale per
# channel.  A PreparedWeight makes those forms straight from the v1 buffers -- at load time through
# prepare_weight() / prepare_model(), otherwise at the first call -- and keeps only the form that is used: a form
# that was made ahead and never asked for is dropped as soon as the other one is.  It hangs on the v1 tensor
# object itself (an attribute, so it lives exactly as long as that tensor and no address or version counter has
# to be trusted to identify it); in-place writes to the v1 tensors are noticed where the tensor counts them.


def _version_of(t: torch.Tensor):
    # Inference tensors count no versions (reading ._version raises) although code under torch.inference_mode() may
    # write them in place (copy_, load_state_dict into existing buffers).  Such a write is invisible here: whoever
    # makes one calls release_prepared(tensor, concatenations=True); prepare_weight / prepare_model -- what the loader
    # and enable_vdm_kernel_mode run -- do not trust a form kept on an inference tensor and make it anew.
    return None if t.is_inference() else t._version


class PreparedWeight:
    """Operand forms of one packed weight, or of the row-concatenation of several (Wq|Wk|Wv): every 128-row block
    of either form is self-contained, so the concatenation's forms are the parts' forms one after the other."""

    def __init__(self, parts):
        parts = [(q, s) for q, s in parts]
        q0 = parts[0][0]
        self.K = q0.shape[1] * 2
        self.rows = [q.shape[0] for q, _ in parts]
        self.N = sum(self.rows)
        self.device = q0.device
        for q, s in parts:
            _check_device_tensor(q, "qweight", torch.uint8)
            _check_device_tensor(s, "wscales", torch.float16)
            _require(q.dim() == 2 and q.shape[1] * 2 == self.K and q.device == self.device, "the parts of a packed weight must agree in K and device")
            _require(tuple(s.shape) == (q.shape[0], self.K // WARP_K), "wscales shape must be [N, K/64]")
        self._parts = [(weakref.ref(q), weakref.ref(s)) for q, s in parts]
        self._versions = [(_version_of(q), _version_of(s)) for q, s in parts]
        self.native: Optional[torch.Tensor] = None
        self.bf6: Optional[torch.Tensor] = None
        self._used = {"native": False, "bf6": False}
        # name of a form -> (event recorded behind the kernels that made it, the stream they ran on, streams that have
        # waited for the event since): a form made lazily inside a forward is made on whatever stream is current
        # then, and a later call on another stream has to be ordered behind it
        self._ready: Dict[str, tuple] = {}
        lib = _load_ext()
        with torch.cuda.device(self.device):
            self.wscale = torch.empty((self.N,), dtype=torch.float16, device=self.device)
            row = 0
            for (q, s), n in zip(parts, self.rows):
                _lib.check(lib.vdmq_wscale_v1_to_plain(s.data_ptr(), self.wscale[row:].data_ptr(), n, self.K, _stream(self.device)))
                row += n
            self._made("wscale")

    def _made(self, name: str) -> None:
        stream = torch.cuda.current_stream(self.device)
        if torch.cuda.is_current_stream_capturing():
            return  # inside a graph the capture orders the work; nothing outside the graph may depend on it
        event = torch.cuda.Event()
        event.record(stream)
        self._ready[name] = (event, stream.cuda_stream, set())

    def _order_behind(self, name: str) -> None:
        """Make the current stream wait for the kernels that made form ``name`` if they ran on another stream."""
        ready = self._ready.get(name)
        if ready is None:
            return
        event, made_on, waited = ready
        stream = torch.cuda.current_stream(self.device)
        if stream.cuda_stream == made_on or stream.cuda_stream in waited:
            return
        if torch.cuda.is_current_stream_capturing():
            return  # (torch.cuda.graph synchronises the device before it starts capturing)
        stream.wait_event(event)
        waited.add(stream.cuda_stream)

    def adopt(self, form: str, tensor: torch.Tensor) -> None:
        """Take ``tensor``, just made on the current stream, as this weight's ``form`` ("native" or "bf6")."""
        setattr(self, form, tensor)
        self._made(form)

    def matches(self, parts) -> bool:
        if len(parts) != len(self._parts):
            return False
        for (rq, rs), (vq, vs), (q, s) in zip(self._parts, self._versions, parts):
            if rq() is not q or rs() is not s or _version_of(q) != vq or _version_of(s) != vs:
                return False
        return True

    def current(self) -> bool:
        """The packed tensors still exist and have not been written since."""
        parts = [(rq(), rs()) for rq, rs in self._parts]
        return all(q is not None and s is not None for q, s in parts) and self.matches(parts)

    def sources(self):
        """The packed v1 tensors this weight was made from: ``[(qweight, wscales), ...]``."""
        return self._sources()

    def _sources(self):
        parts = [(rq(), rs()) for rq, rs in self._parts]
        if any(q is None for q, _ in parts):
            raise _lib.VdmqError("the packed weight tensors of this prepared weight are gone")
        return parts

    def _build(self, form: str) -> torch.Tensor:
        lib = _load_ext()
        K = self.K
        for q, _ in self._sources():
            ensure_v1(q)  # (freed by release_v1: comes back from the form that is there)
        with torch.cuda.device(self.device):
            s = _stream(self.device)
            if form == "bf6":
                out = torch.empty((int(lib.vdmq_bf6_bytes(self.N, K)),), dtype=torch.uint8, device=self.device)
                row_bytes = int(lib.vdmq_bf6_bytes(32, K)) // 32
                convert = lib.vdmq_weight_v1_to_bf6
            else:
                out = torch.empty((self.N, k_padded(K) // 2), dtype=torch.uint8, device=self.device)
                row_bytes = k_padded(K) // 2
                convert = lib.vdmq_weight_v1_to_native
            flat, row = out.view(-1), 0
            for (q, _), n in zip(self._sources(), self.rows):
                _lib.check(convert(q.data_ptr(), flat[row * row_bytes:].data_ptr(), n, K, s))
                row += n
            setattr(self, form, out)
            self._made(form)
        return out

    # -- the v1 weight buffers' storage: with a prepared form resident the kernels never read them again; they only
    # remain what state_dict() returns.  release_v1 frees their memory (the tensor objects keep shape, dtype and
    # device: they are the module's buffers), restore_v1 brings the bytes back from the prepared form.
    def release_v1(self) -> int:
        """Free the storage of the packed v1 weight tensors this weight was made from (not the small scale tensors);
        returns the bytes freed.  Needs a prepared form to restore from, and tensors that own their whole storage."""
        if self.bf6 is None and self.native is None:
            return 0
        freed = 0
        for index, (q, _) in enumerate(self._sources()):
            storage = q.untyped_storage()
            if "_vdmq_v1_released" in q.__dict__ or q.storage_offset() != 0 or storage.nbytes() != q.numel() * q.element_size():
                continue
            freed += storage.nbytes()
            self._order_behind("bf6" if self.bf6 is not None else "native")
            q.__dict__["_vdmq_v1_released"] = (self, index)  # (keeps this weight, i.e. the only copy of the integers, alive)
            storage.resize_(0)
        return freed

    def restore_v1(self, index: int) -> None:
        q = self._sources()[index][0]
        if q.__dict__.get("_vdmq_v1_released", (None,))[0] is not self:
            return
        lib = _load_ext()
        bf6 = self.bf6 is not None
        form = self.bf6 if bf6 else self.native
        if form is None:
            raise _lib.VdmqError("the prepared form this packed weight was to be restored from is gone")
        row_bytes = int(lib.vdmq_bf6_bytes(32, self.K)) // 32 if bf6 else k_padded(self.K) // 2
        row = sum(self.rows[:index])
        with torch.cuda.device(self.device):
            q.untyped_storage().resize_(q.numel() * q.element_size())
            self._order_behind("bf6" if bf6 else "native")
            convert = lib.vdmq_bf6_to_weight_v1 if bf6 else lib.vdmq_weight_native_to_v1
            _lib.check(convert(form.view(-1)[row * row_bytes:].data_ptr(), q.data_ptr(), self.rows[index], self.K, _stream(self.device)))
        del q.__dict__["_vdmq_v1_released"]

    def operand(self, bf6: bool, eager: bool = False) -> torch.Tensor:
        """The weights as bf6 blocks (``bf6``) or native int4 rows.  ``eager``: made ahead of use -- it does not count
        as a use and drops nothing."""
        form, other = ("bf6", "native") if bf6 else ("native", "bf6")
        if getattr(self, form) is None:
            self._build(form)
        if not eager:
            self._used[form] = True
            if getattr(self, other) is not None and not self._used[other]:
                setattr(self, other, None)  # made ahead for a call pattern that did not come
                self._ready.pop(other, None)
        self._order_behind("wscale")
        self._order_behind(form)
        return getattr(self, form)

    def extra_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.native, self.bf6, self.wscale) if t is not None)


def ensure_v1(qweight: torch.Tensor) -> None:
    """Bring back the bytes of a packed v1 weight whose storage release_v1_storage freed (a no-op otherwise).  A
    projection's buffer that is a view of its attention module's concatenation comes back with that."""
    owner = qweight.__dict__.get("_vdmq_v1_owner")
    if owner is not None and owner() is not None:
        qweight = owner()
    released = qweight.__dict__.get("_vdmq_v1_released")
    if released is not None:
        released[0].restore_v1(released[1])


def _restore_before_state_dict(module, prefix, keep_vars) -> None:
    ensure_v1(module.vdm_weight_packed)


def release_v1_storage(model) -> int:
    """Free the memory of every packed v1 weight buffer of ``model`` whose prepared form is resident: 3/4 (bf6
    blocks) or 1/2 (native rows) byte per weight stays, instead of 1/2 more beside it.  The buffers remain the
    modules' ``vdm_weight_packed`` (same objects, shape, dtype, device); ``state_dict()`` -- and with it
    ``save_packed_checkpoint`` -- brings the bytes back first (vdmq_bf6_to_weight_v1 / vdmq_weight_native_to_v1
    reproduce them exactly).  Call ``restore_v1_storage(model)`` before anything else that reads or moves the
    buffers (``model.to(...)``, ``load_state_dict``).  Returns the bytes freed."""
    freed = 0
    for module in model.modules():
        q = getattr(module, "vdm_weight_packed", None)
        if q is None or not q.is_cuda:
            continue
        owner = q.__dict__.get("_vdmq_v1_owner")
        holder = owner() if owner is not None and owner() is not None else q
        for pw in holder.__dict__.get(_ATTR, []):
            if pw.current() and len(pw.rows) == 1:
                freed += pw.release_v1()
                break
        if "_vdmq_v1_released" in holder.__dict__ and not hasattr(module, "_vdmq_v1_hook"):
            module._vdmq_v1_hook = module.register_state_dict_pre_hook(_restore_before_state_dict)
    return freed


def restore_v1_storage(model) -> None:
    for module in model.modules():
        q = getattr(module, "vdm_weight_packed", None)
        if q is not None:
            ensure_v1(q)


_ATTR = "_vdmq_prepared"


def _prepared(parts) -> PreparedWeight:
    """The PreparedWeight of a packed weight given as ``[(qweight, wscales), ...]`` (one pair, or the pairs whose
    rows are concatenated), kept on the first pair's qweight tensor."""
    holder = parts[0][0]
    kept = holder.__dict__.get(_ATTR)
    if kept is not None:
        for pw in kept:
            if pw.matches(parts):
                return pw
        kept[:] = [pw for pw in kept if pw.current()]  # drop what was overwritten since
    pw = PreparedWeight(parts)
    holder.__dict__.setdefault(_ATTR, []).append(pw)
    return pw


def _prepared_weight(qweight: torch.Tensor, wscales: torch.Tensor) -> PreparedWeight:
    if not (qweight.is_contiguous() and wscales.is_contiguous()):
        # a fresh contiguous copy per call would be relaid per call: keep the copy with the tensor it came from
        kept = qweight.__dict__.get("_vdmq_contiguous")
        if kept is None or kept[0]() is not wscales or kept[1] != (_version_of(qweight), _version_of(wscales)):
            kept = (weakref.ref(wscales), (_version_of(qweight), _version_of(wscales)), qweight.contiguous(), wscales.contiguous())
            qweight.__dict__["_vdmq_contiguous"] = kept
        qweight, wscales = kept[2], kept[3]
    return _prepared([(qweight, wscales)])


def prepare_weight(qweight: torch.Tensor, wscales: torch.Tensor, tokens: Optional[int] = None, path: Optional[str] = None) -> PreparedWeight:
    """Relayout a packed weight now (load time, a known stream) instead of at its first call.  ``tokens``: the number
    of rows its calls will have, passed on to the library's rule for the matrix path under "auto" (which at present
    looks at the row length only; default: a video-sized sequence)."""
    if qweight.is_inference():
        release_prepared(qweight, concatenations=True)  # written in place since? not visible: see _version_of
    pw = _prepared_weight(qweight, wscales)
    pw.operand(_use_bf6(32768 if tokens is None else int(tokens), pw.N, pw.K, path=path), eager=True)
    return pw


def prepare_model(model, tokens: Optional[int] = None, path: Optional[str] = None) -> int:
    """prepare_weight for every module of ``model`` that holds packed buffers and runs in kernel mode (the place the
    reference attaches those buffers: packed_checkpoint.py:102-148, quant_linear.py:146-160).  Attention modules
    marked for the fused QKV / KV path get the concatenated form instead of one per projection.  Returns the bytes
    of HBM the prepared forms take beside the v1 buffers."""
    from ..fused_qkv import concatenated, fused_parts

    done, total = set(), 0
    for module in model.modules():
        for names in fused_parts(module):
            layers = [getattr(module, n) for n in names]
            if not all(l.vdm_weight_packed.is_cuda for l in layers):
                continue
            total += prepare_weight(*concatenated(module, names), tokens, path).extra_bytes()
            done.update(id(l) for l in layers)
    for module in model.modules():
        if id(module) in done or not getattr(module, "use_vdm_kernel", False) or getattr(module, "vdm_weight_packed", None) is None:
            continue
        if not module.vdm_weight_packed.is_cuda:
            continue
        total += prepare_weight(module.vdm_weight_packed, module.vdm_weight_scale_packed, tokens, path).extra_bytes()
    return total


def release_prepared(qweight: torch.Tensor, concatenations: bool = False) -> None:
    """Drop the prepared forms kept with ``qweight`` for itself (and, with ``concatenations``, for concatenations it
    leads): a projection that is only ever used through its attention module's fused weight needs none of its own."""
    kept = qweight.__dict__.get(_ATTR)
    if kept is not None:
        ensure_v1(qweight)  # a form about to go may hold the only copy of the integers
        kept[:] = [pw for pw in kept if len(pw.rows) > 1 and not concatenations]


def _native_weights(qweight: torch.Tensor, wscales: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """(native int4 rows, plain fp16 channel scales) of a packed weight."""
    pw = _prepared_weight(qweight, wscales)
    return pw.operand(False), pw.wscale


# ------------------------------------------------- which matrix instructions run the GEMM
# "int8": v_mfma_i32_32x32x32_i8 on nibbles widened in registers.  "bf6": v_mfma_f32_32x32x64_f8f6f4 on 6-bit
# floats (twice the rate, no widening work; every int4 value q is held as the E3M2 float q / 16, exactly, and the
# fp32 accumulation of the products is exact too).
# Both give bit-identical results.  "auto" asks the library (vdmq_bf6_pays: bf6 from a row length of 1280 on, whatever
# the other sizes -- its GEMM has a tile configuration for small problems, and only its quantizer is the slower one on
# short rows).
_MATRIX_PATH = os.environ.get("VDMQ_MATRIX_PATH", "auto")


def set_matrix_path(name: str) -> None:
    global _MATRIX_PATH
    if name not in ("auto", "int8", "bf6"):
        raise ValueError("matrix path must be 'auto', 'int8' or 'bf6'")
    _MATRIX_PATH = name


def matrix_path() -> str:
    return _MATRIX_PATH


def _use_bf6(M: int, N: int, K: int, out_dtype: torch.dtype = torch.float16, path: Optional[str] = None) -> bool:
    path = _MATRIX_PATH if path is None else path
    if path == "int8" or M == 0:
        return False
    if path == "bf6":
        return True
    return bool(_load_ext().vdmq_bf6_pays(M, N, K))


def _to_bf6(native: torch.Tensor, rows: int, K: int) -> torch.Tensor:
    lib = _load_ext()
    blocks = torch.empty((int(lib.vdmq_bf6_bytes(rows, K)),), dtype=torch.uint8, device=native.device)
    if rows:
        _lib.check(lib.vdmq_native_to_bf6(native.data_ptr(), rows, K, blocks.data_ptr(), _stream(native.device)))
    return blocks


def _quantize_for_gemm(x_2d: torch.Tensor, clip_ratio: float, act_code: int, bf6: bool, ln_args: Optional[tuple] = None):
    """Quantize the rows of ``x_2d`` (optionally through a fused activation, or the fused LayerNorm described by
    ``ln_args`` = the leading arguments of vdmq_quantize_act_ln) into the operand form of the chosen matrix path:
    bf6 blocks or native int4 rows.  Returns ``(operand, scales)``.  Must run under ``torch.cuda.device(...)``."""
    lib = _load_ext()
    M, K = x_2d.shape
    dev = x_2d.device
    s = _stream(dev)
    scales = torch.empty((M,), dtype=torch.float16, device=dev)
    direct = bf6 and K <= 16384  # the quantizer writes bf6 blocks itself
    if direct:
        op = torch.empty((int(lib.vdmq_bf6_bytes(M, K)),), dtype=torch.uint8, device=dev)
    else:
        op = torch.empty((M, k_padded(K) // 2), dtype=torch.uint8, device=dev)
    if ln_args is not None:
        fn = lib.vdmq_quantize_act_ln_bf6 if direct else lib.vdmq_quantize_act_ln
        _lib.check(fn(*ln_args, float(clip_ratio), op.data_ptr(), scales.data_ptr(), s))
    else:
        fn = lib.vdmq_quantize_act_bf6 if direct else lib.vdmq_quantize_act_ex
        _lib.check(fn(x_2d.data_ptr(), M, K, x_2d.stride(0), float(clip_ratio), act_code, op.data_ptr(), scales.data_ptr(), s))
    if bf6 and not direct:
        op = _to_bf6(op, M, K)
    return op, scales


def _gemm_dispatch(operand: torch.Tensor, scales: torch.Tensor, bf6: bool, weight: PreparedWeight,
                   bias: Optional[torch.Tensor], out: torch.Tensor, K: int, gate: Optional[torch.Tensor] = None, rows_per_gate: int = 1,
                   residual: Optional[torch.Tensor] = None) -> None:
    """GEMM + epilogue on a quantized activation (bf6 blocks if ``bf6`` else native rows) into ``out`` [M, N], or,
    for an ``out`` of shape [N / cols, M, cols], into N / cols separate matrices (vdmq_gemm_w4a4_split).
    Must run under ``torch.cuda.device(out.device)``."""
    lib = _load_ext()
    s = _stream(out.device)
    bias_p = None if bias is None else bias.data_ptr()
    if out.dim() == 3:
        _require(gate is None and residual is None and out.dtype == torch.float16, "a split output takes neither gate nor residual and is fp16")
        parts, M, cols = out.shape
        fn = lib.vdmq_gemm_w4a4_bf6_split if bf6 else lib.vdmq_gemm_w4a4_split
        _lib.check(fn(operand.data_ptr(), scales.data_ptr(), weight.operand(bf6).data_ptr(), weight.wscale.data_ptr(), bias_p, out.data_ptr(),
                      M, parts * cols, K, out.stride(1), cols, out.stride(0), s))
        return
    M, N = out.shape
    gate_p, ldg = (None, 0) if gate is None else (gate.data_ptr(), gate.stride(0))
    res_p, ldr = (None, 0) if residual is None else (residual.data_ptr(), residual.stride(0))
    w, wscale = weight.operand(bf6), weight.wscale
    code = _lib.VDMQ_OUT_F16 if out.dtype == torch.float16 else _lib.VDMQ_OUT_BF16
    if bf6:
        _lib.check(lib.vdmq_gemm_w4a4_bf6_ex(operand.data_ptr(), scales.data_ptr(), w.data_ptr(), wscale.data_ptr(), bias_p, gate_p, ldg,
                                             rows_per_gate, res_p, ldr, out.data_ptr(), code, M, N, K, out.stride(0), s))
        return
    _lib.check(lib.vdmq_gemm_w4a4_ex(operand.data_ptr(), scales.data_ptr(), w.data_ptr(), wscale.data_ptr(), bias_p, gate_p, ldg,
                                     rows_per_gate, res_p, ldr, out.data_ptr(), code, M, N, K, out.stride(0), s))


# -------------------------------------------------------------- public API

def pack_weight_with_scale(weight: torch.Tensor, channel_scale: torch.Tensor):
    """Pack fp weights with caller-provided per-channel scales.

    Returns ``(qweight u8 [N, K/2] v1, packed_scales fp16 [N, K/64] v1,
    channel_scales fp16 [N])`` like vdm_w4a4.py:209-214 /
    vdm_w4a4_kernel.cu:697-728.
    """
    lib = _load_ext()
    weight_h = weight.detach().half().contiguous()
    scale_h = channel_scale.detach().view(-1).half().contiguous().to(weight_h.device)
    _check_device_tensor(weight_h, "weight", torch.float16)
    _require(weight_h.dim() == 2, "weight must be [N, K]")
    N, K = weight_h.shape
    _require(scale_h.numel() == N, "channel_scales length must equal N")
    _require(N % BLOCK_N == 0, f"N must be a multiple of {BLOCK_N}")
    _require(K % WARP_K == 0, f"K must be a multiple of {WARP_K}")
    dev = weight_h.device
    with torch.cuda.device(dev):
        s = _stream(dev)
        native = torch.empty((N, k_padded(K) // 2), dtype=torch.uint8, device=dev)
        qweight = torch.empty((N, K // 2), dtype=torch.uint8, device=dev)
        packed_scales = torch.empty((N, K // WARP_K), dtype=torch.float16, device=dev)
        _lib.check(lib.vdmq_quantize_weight_native(weight_h.data_ptr(), scale_h.data_ptr(), native.data_ptr(), N, K, s))
        _lib.check(lib.vdmq_weight_native_to_v1(native.data_ptr(), qweight.data_ptr(), N, K, s))
        _lib.check(lib.vdmq_wscale_plain_to_v1(scale_h.data_ptr(), packed_scales.data_ptr(), N, K, s))
    # the native form is already at hand: a first GEMM on the int8 path needs no relayout (an eager form: the bf6
    # path, if that is what the calls take, drops it)
    _prepared([(qweight, packed_scales)]).adopt("native", native)
    return qweight, packed_scales, scale_h


def quantize_weight_per_channel(weight: torch.Tensor):
    """Derive per-channel scales (absmax/7, clip 1) and pack
    (vdm_w4a4.py:217-219 / vdm_w4a4_kernel.cu:730-763)."""
    lib = _load_ext()
    weight_h = weight.detach().half().contiguous()
    _check_device_tensor(weight_h, "weight", torch.float16)
    _require(weight_h.dim() == 2, "weight must be [N, K]")
    N, K = weight_h.shape
    _require(N % BLOCK_N == 0, f"N must be a multiple of {BLOCK_N}")
    _require(K % WARP_K == 0, f"K must be a multiple of {WARP_K}")
    with torch.cuda.device(weight_h.device):
        scales = torch.empty((N,), dtype=torch.float16, device=weight_h.device)
        _lib.check(lib.vdmq_row_scale(weight_h.data_ptr(), N, K, 1.0, scales.data_ptr(), _stream(weight_h.device)))
    return pack_weight_with_scale(weight_h, scales)


_ACTIVATIONS = {None: _lib.VDMQ_ACT_NONE, "none": _lib.VDMQ_ACT_NONE, "gelu_tanh": _lib.VDMQ_ACT_GELU_TANH}


def _act_code(act: Optional[str]) -> int:
    if act not in _ACTIVATIONS:
        raise ValueError(f"unknown activation {act!r}; expected one of {sorted(k for k in _ACTIVATIONS if k)}")
    return _ACTIVATIONS[act]


def _linear_2d(x_2d: torch.Tensor, weight: PreparedWeight, bias: Optional[torch.Tensor], clip_ratio: float,
               out_dtype: torch.dtype = torch.float16, act: Optional[str] = None, split_cols: Optional[int] = None) -> torch.Tensor:
    """[M, N], or [N / split_cols, M, split_cols] with ``split_cols`` (each part a contiguous matrix)."""
    _load_ext()  # raises when the library is missing
    M, K = x_2d.shape
    N = weight.N
    dev = x_2d.device
    _require(weight.device == dev, "weights and input must be on the same device")
    if bias is not None:
        _check_device_tensor(bias, "bias", torch.float16)
        _require(bias.dim() == 1, "bias must be [N]")
        _require(bias.numel() == N, "bias length must equal N")
    if split_cols is not None and (split_cols <= 0 or split_cols % 64 != 0 or N % split_cols != 0):
        raise ValueError(f"split_cols must be a positive multiple of 64 that divides N={N} (got {split_cols})")
    with torch.cuda.device(dev):
        shape = (M, N) if split_cols is None else (N // split_cols, M, split_cols)
        out = torch.empty(shape, dtype=out_dtype, device=dev)
        if M == 0:
            return out
        bf6 = _use_bf6(M, N, K, out_dtype)
        operand, scales = _quantize_for_gemm(x_2d, clip_ratio, _act_code(act), bf6)
        _gemm_dispatch(operand, scales, bf6, weight, bias, out, K)
    return out


def linear_vdm_w4a4(
    x: torch.Tensor,
    qweight: torch.Tensor,
    wscales: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    clip_ratio: float = 1.0,
    bias_half: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """W4A4 linear: dynamic per-token A4 quantization of ``x``, int4 x int4 GEMM
    against the packed weights, per-token x per-channel scale and fp16 bias.
    Signature and semantics of vdm_w4a4.py:222-244; the output is always fp16."""
    _load_ext()
    x_2d, orig_shape = _as_2d_half_contiguous(x)
    _check_linear_shapes(x_2d, qweight, wscales)
    _require(x_2d.is_cuda, "input must be a CUDA tensor")
    return _linear_prepared(x_2d, _prepared_weight(qweight, wscales), bias_half if bias_half is not None else bias, clip_ratio).view(*orig_shape, -1)


def linear_vdm_w4a4_prepared(x: torch.Tensor, weight: PreparedWeight, bias_half: Optional[torch.Tensor] = None,
                             clip_ratio: float = 1.0, split_cols: Optional[int] = None) -> torch.Tensor:
    """``linear_vdm_w4a4`` on a weight that is already in the kernels' form -- what the fused QKV / KV dispatch calls
    with the concatenated weight of an attention module (no counterpart in the reference, which passes concatenated
    v1 buffers to the same function).  ``split_cols``: the N output columns are written as N / split_cols separate
    contiguous tensors, returned stacked as ``[N / split_cols, ..., split_cols]`` -- the bits of
    ``out.split(split_cols, -1)``, without the strided views (the GEMM epilogue writes them in place)."""
    _load_ext()
    x_2d, orig_shape = _as_2d_half_contiguous(x)
    if weight.K != x_2d.shape[1]:
        raise ValueError("qweight shape must be [N, K/2]")
    _require(x_2d.is_cuda, "input must be a CUDA tensor")
    out = _linear_prepared(x_2d, weight, bias_half, clip_ratio, split_cols)
    return out.view(*orig_shape, -1) if split_cols is None else out.view(out.shape[0], *orig_shape, split_cols)


def _linear_prepared(x_2d: torch.Tensor, weight: PreparedWeight, bias: Optional[torch.Tensor], clip_ratio: float,
                     split_cols: Optional[int] = None) -> torch.Tensor:
    if bias is not None:
        bias = bias.half().contiguous().view(-1)
    return _linear_2d(x_2d, weight, bias, clip_ratio, split_cols=split_cols)


def quantize_activation_per_token(x: torch.Tensor, clip_ratio: float = 1.0):
    """Returns ``(qact u8 [ceil(M,256), K/2], ascales fp16 [ceil(M,256), K/64],
    act_scales fp16 [M])`` in the reference's v1 layouts
    (vdm_w4a4.py:247-250 / vdm_w4a4_kernel.cu:840-874)."""
    lib = _load_ext()
    x_2d, _ = _as_2d_half_contiguous(x)
    _check_device_tensor(x_2d, "input", torch.float16)
    M, K = x_2d.shape
    _require(K % WARP_K == 0, f"K must be a multiple of {WARP_K}")
    PM = (M + BLOCK_M - 1) // BLOCK_M * BLOCK_M
    dev = x_2d.device
    with torch.cuda.device(dev):
        s = _stream(dev)
        native = torch.empty((M, k_padded(K) // 2), dtype=torch.uint8, device=dev)
        act_scales = torch.empty((M,), dtype=torch.float16, device=dev)
        qact = torch.empty((PM, K // 2), dtype=torch.uint8, device=dev)
        ascales = torch.empty((PM, K // WARP_K), dtype=torch.float16, device=dev)
        _lib.check(lib.vdmq_quantize_act(x_2d.data_ptr(), M, K, x_2d.stride(0), float(clip_ratio), native.data_ptr(),
                                         act_scales.data_ptr(), s))
        _lib.check(lib.vdmq_act_native_to_v1(native.data_ptr(), act_scales.data_ptr(), M, K, qact.data_ptr(), ascales.data_ptr(), s))
    return qact, ascales, act_scales


def quantize_activation_native(x: torch.Tensor, clip_ratio: float = 1.0, act: Optional[str] = None):
    """The quantizer's own output: ``(qact u8 [M, Kp/2] row-major, scales fp16 [M])``.
    ``act="gelu_tanh"`` quantizes ``gelu_tanh(x)`` instead of ``x`` in the same pass."""
    lib = _load_ext()
    x_2d, _ = _as_2d_half_contiguous(x)
    _check_device_tensor(x_2d, "input", torch.float16)
    M, K = x_2d.shape
    _require(K % WARP_K == 0, f"K must be a multiple of {WARP_K}")
    dev = x_2d.device
    with torch.cuda.device(dev):
        native = torch.empty((M, k_padded(K) // 2), dtype=torch.uint8, device=dev)
        act_scales = torch.empty((M,), dtype=torch.float16, device=dev)
        _lib.check(lib.vdmq_quantize_act_ex(x_2d.data_ptr(), M, K, x_2d.stride(0), float(clip_ratio), _act_code(act),
                                            native.data_ptr(), act_scales.data_ptr(), _stream(dev)))
    return native, act_scales


def quantize_activation_bf6(x: torch.Tensor, clip_ratio: float = 1.0, act: Optional[str] = None):
    """The quantizer writing the bf6 GEMM's operand form directly: ``(blocks u8 [vdmq_bf6_bytes(M, K)], scales fp16 [M])``
    -- the same integers and scales as ``quantize_activation_native``; rows of the last 32-row block beyond M are unspecified."""
    _load_ext()
    x_2d, _ = _as_2d_half_contiguous(x)
    _check_device_tensor(x_2d, "input", torch.float16)
    _require(x_2d.shape[1] % WARP_K == 0, f"K must be a multiple of {WARP_K}")
    with torch.cuda.device(x_2d.device):
        return _quantize_for_gemm(x_2d, clip_ratio, _act_code(act), True)


def linear_prequantized(qact: torch.Tensor, ascales: torch.Tensor, qweight: torch.Tensor, wscales: torch.Tensor) -> torch.Tensor:
    """GEMM only, on v1-layout activations already padded to BLOCK_M rows; no
    bias (vdm_w4a4.py:253-256 / vdm_w4a4_kernel.cu:876-918)."""
    lib = _load_ext()
    qact, ascales = qact.contiguous(), ascales.contiguous()
    qweight, wscales = qweight.contiguous(), wscales.contiguous()
    _check_device_tensor(qact, "qact", torch.uint8)
    _check_device_tensor(ascales, "ascales", torch.float16)
    _check_device_tensor(qweight, "qweight", torch.uint8)
    _check_device_tensor(wscales, "wscales", torch.float16)
    _require(qact.dim() == 2 and ascales.dim() == 2 and qweight.dim() == 2 and wscales.dim() == 2, "all inputs must be 2-D")
    M, K, N = qact.shape[0], qact.shape[1] * 2, qweight.shape[0]
    _require(qweight.shape[1] == K // 2, "qweight second dim must be K / 2")
    _require(K % WARP_K == 0, f"K must be a multiple of {WARP_K}")
    _require(tuple(ascales.shape) == (M, K // WARP_K), "bad ascales shape")
    _require(tuple(wscales.shape) == (N, K // WARP_K), "bad wscales shape")
    _require(M % BLOCK_M == 0, f"M must be a multiple of {BLOCK_M}")
    _require(N % BLOCK_N == 0, f"N must be a multiple of {BLOCK_N}")
    weight = _prepared_weight(qweight, wscales)
    dev = qact.device
    with torch.cuda.device(dev):
        s = _stream(dev)
        out = torch.empty((M, N), dtype=torch.float16, device=dev)
        if M == 0:
            return out
        native = torch.empty((M, k_padded(K) // 2), dtype=torch.uint8, device=dev)
        scales = torch.empty((M,), dtype=torch.float16, device=dev)
        _lib.check(lib.vdmq_act_v1_to_native(qact.data_ptr(), ascales.data_ptr(), M, K, native.data_ptr(), scales.data_ptr(), s))
        bf6 = _use_bf6(M, N, K)
        _gemm_dispatch(_to_bf6(native, M, K) if bf6 else native, scales, bf6, weight, None, out, K)
    return out


def gemm_int32_accumulators(qact_native: torch.Tensor, wq_native: torch.Tensor, K: int, path: Optional[str] = None) -> torch.Tensor:
    """Checker's view: the exact int32 accumulators of the GEMM, [M, N], on the int8 or the bf6 matrix path
    (``path`` None: the one ``matrix_path()`` selects for this shape)."""
    lib = _load_ext()
    M, N = qact_native.shape[0], wq_native.shape[0]
    dev = qact_native.device
    bf6 = path == "bf6" or (path is None and _use_bf6(M, N, K))
    with torch.cuda.device(dev):
        acc = torch.empty((M, N), dtype=torch.int32, device=dev)
        if M and bf6:
            xb, wb = _to_bf6(qact_native, M, K), _to_bf6(wq_native, N, K)
            _lib.check(lib.vdmq_gemm_w4a4_bf6_acc(xb.data_ptr(), wb.data_ptr(), acc.data_ptr(), M, N, K, _stream(dev)))
        elif M:
            _lib.check(lib.vdmq_gemm_w4a4_acc(qact_native.data_ptr(), wq_native.data_ptr(), acc.data_ptr(), M, N, K, _stream(dev)))
    return acc


def bf6_blocks(native: torch.Tensor, K: int) -> torch.Tensor:
    """The bf6 block form (see include/vdmq.h) of a native int4 buffer, for inspection."""
    with torch.cuda.device(native.device):
        return _to_bf6(native.contiguous(), native.shape[0], K)


def linear_vdm_w4a4_qkv(
    x: torch.Tensor,
    q_weight_packed: torch.Tensor,
    q_weight_scale: torch.Tensor,
    k_weight_packed: torch.Tensor,
    k_weight_scale: torch.Tensor,
    v_weight_packed: torch.Tensor,
    v_weight_scale: torch.Tensor,
    q_bias: Optional[torch.Tensor] = None,
    k_bias: Optional[torch.Tensor] = None,
    v_bias: Optional[torch.Tensor] = None,
    clip_ratio: float = 1.0,
    w_qkv_packed: Optional[torch.Tensor] = None,
    w_qkv_scale: Optional[torch.Tensor] = None,
    qkv_bias_half: Optional[torch.Tensor] = None,
    contiguous_outputs: bool = False,
):
    """Fused QKV: one activation quantization and one GEMM against the row-concatenated Wq|Wk|Wv; returns three
    views of one [..., 3N] tensor.  Signature, argument handling (cached concatenation if given, zeros for missing
    biases, ``split(n)``) and results are fixed by the reference's function of the same name (vdm_w4a4.py:259-298),
    which this follows step by step.  Without the cached concatenation the reference concatenates the v1 buffers on
    every call; here the three buffers are relaid once into one operand (every 128-row block of a v1 buffer is
    self-contained, so the concatenation's operand is the parts' operands one after the other) and that is kept.
    ``contiguous_outputs`` (not in the reference): q, k and v are written by the GEMM epilogue as three contiguous
    tensors instead of strided views of one -- the same bits."""
    if w_qkv_packed is None or w_qkv_scale is None:
        weight = _prepared([(q_weight_packed.contiguous(), q_weight_scale.contiguous()), (k_weight_packed.contiguous(), k_weight_scale.contiguous()),
                            (v_weight_packed.contiguous(), v_weight_scale.contiguous())])
    else:
        weight = _prepared_weight(w_qkv_packed, w_qkv_scale)
    n = q_weight_packed.shape[0]
    if qkv_bias_half is None and (q_bias is not None or k_bias is not None or v_bias is not None):
        device = q_weight_packed.device
        parts = [b.half().contiguous() if b is not None else torch.zeros(n, dtype=torch.float16, device=device) for b in (q_bias, k_bias, v_bias)]
        qkv_bias_half = torch.cat(parts, dim=0)
    _load_ext()
    x_2d, orig_shape = _as_2d_half_contiguous(x)
    _check_packed_weight(q_weight_packed, q_weight_scale, x_2d.shape[1])
    _require(x_2d.is_cuda, "input must be a CUDA tensor")
    if contiguous_outputs:
        return _linear_prepared(x_2d, weight, qkv_bias_half, clip_ratio, split_cols=n).view(3, *orig_shape, n).unbind(0)
    qkv = _linear_prepared(x_2d, weight, qkv_bias_half, clip_ratio).view(*orig_shape, -1)
    return qkv.split(n, dim=-1)
