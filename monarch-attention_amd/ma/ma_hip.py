"""Host side of the HIP implementation: marshals torch tensors into the C ABI.

``monarch_attention_hip`` has the signature of the reference's implementation
functions (``MonarchAttentionFn``, ma/monarch_attention.py:11-13; the torch
one is ``monarch_attention_torch``, ma/ma_torch.py:65-73):

    fn(q, k, v, attn_mask, T, B, pre_pad) -> Tensor

q, k ``(E, H, N, D)``; v ``(E, H, N, Dv)`` (its dtype is the output dtype and
may differ from q/k, as in ``get_matrix``); ``attn_mask`` ``(E, N)`` bool /
int / float, truthy = keep, or ``None``.  Inputs may be arbitrary strided views
with a contiguous last dimension (models pass permuted ``(E, N, H, D)``
buffers); nothing is padded or copied on the host - the kernels apply the
reference's zero padding (ma/ma_torch.py:81-86) by index arithmetic and write
only the N real rows.  PyTorch provides the device buffers (output, workspace)
and the stream; all arithmetic happens in libma_hip.so.
"""
from __future__ import annotations

import os
import threading

import torch

from . import _hip_lib as L

Tensor = torch.Tensor

_DTYPES = {torch.float32: L.MA_F32, torch.float16: L.MA_F16, torch.bfloat16: L.MA_BF16}
_MASK_DTYPES = {torch.bool: L.MA_MASK_U8, torch.uint8: L.MA_MASK_U8, torch.int8: L.MA_MASK_U8, torch.int16: L.MA_MASK_I16,
                torch.int32: L.MA_MASK_I32, torch.int64: L.MA_MASK_I64, torch.float16: L.MA_MASK_F16,
                torch.bfloat16: L.MA_MASK_BF16, torch.float32: L.MA_MASK_F32, torch.float64: L.MA_MASK_F64}

# default variant of monarch_attention_hip; tests and the benchmark switch it
# per call through the `variant` keyword
DEFAULT_VARIANT = "auto"

# Does this process own the GPU while its forward calls run - no other stream,
# thread or process competing for compute units?  Only then may 'auto' resolve
# to the 'fused' kernel, whose workgroups wait for each other and so must all be
# on the device together (MA_FLAG_DEVICE_EXCLUSIVE).  Off unless the environment
# says MA_HIP_DEVICE_EXCLUSIVE=1 or the application sets this attribute; 'auto'
# then stays with kernels that make progress beside any other work.
DEVICE_EXCLUSIVE = os.environ.get("MA_HIP_DEVICE_EXCLUSIVE", "") not in ("", "0")

# One workspace per (device, stream), grown on demand and reused call after
# call: calls on one stream are ordered, so they can share it.  It is allocated
# zero-filled, and every forward call leaves its sync area in the state the next
# call needs (counters and epochs continuing), which is what
# MA_FLAG_SYNC_READY promises to the library.
#
# The one-launch kernels (fused, chained) wait for each other's workgroups with
# bounded waits; a wait that runs out raises a sticky error word in the
# workspace and the workgroup writes NaN instead of results.  The kernel stores
# the same code into a word of pinned host memory that belongs to the workspace
# (ma_fwd_params.error_word), and EVERY call on the workspace looks at that word
# first - a plain host read, nothing is copied or synchronised: a failed call is
# reported by a RuntimeError from the first later call that finds the word set
# (at the latest the first call after the failed call's work has completed), the
# sync area is cleared again, and the call after that is a normal one.
_TEST_FLAGS = 0            # extra ma_fwd_params.flags for the failure-path tests (MA_FLAG_TEST_NO_SPIN)
_SYNCING = (L.VARIANTS["fused"], L.VARIANTS["chained"])


class _Workspace:
    def __init__(self, device: torch.device, nbytes: int):
        self.err_host = torch.zeros(1, dtype=torch.int32, pin_memory=True)
        self.err = self.err_host.numpy()          # the same word, read without a torch call
        self.err_ptr = self.err_host.data_ptr()
        self.dirty = False      # the sync area must be cleared before the next one-launch kernel
        self.resize(device, nbytes)

    def resize(self, device: torch.device, nbytes: int) -> None:
        self.buf = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        self.ptr, self.nbytes = self.buf.data_ptr(), self.buf.numel()


_WORKSPACES: dict[tuple[int, int], _Workspace] = {}


def _workspace(device: torch.device, stream_ptr: int, nbytes: int) -> _Workspace:
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_ptr)
    w = _WORKSPACES.get(key)
    if w is None:
        w = _WORKSPACES[key] = _Workspace(device, nbytes)
    elif w.nbytes < nbytes:
        # calls on this stream that still use the old buffer are ahead of everything queued from here on,
        # and the caching allocator hands a freed block to other streams only after that work is done
        w.resize(device, nbytes)
    return w


def _raise_failed(w: _Workspace) -> None:
    """The host-visible error word of this workspace is set: an earlier call on it failed."""
    code = int(w.err[0])
    w.err[0] = 0
    w.dirty = True
    w.buf[4:8].zero_()      # the word in the workspace is sticky: clear it for the calls to come
    what = {1: "a bounded wait between workgroups ran out",
            2: "workgroups of one head ran on different XCDs (the one-launch kernels rely on ids x, x + 8, ... "
               "sharing an XCD)"}.get(code, f"error word {code}")
    raise RuntimeError(f"monarch_attention_hip: an earlier forward call on this stream failed: {what}; its output "
                       f"holds NaN rows.  The workspace has been reset; pass variant='staged' to avoid the "
                       f"one-launch kernels")


def sync_status() -> int:
    """The sticky error word of the one-launch kernels, over all cached
    workspaces (synchronises the device): 0 = every wait between workgroups was
    satisfied; 1 = a bounded wait ran out (results of that call are invalid);
    2 = a producer ran on another XCD than its consumer (the device does not
    deal workgroup ids to XCDs the way the one-launch kernels are built on)."""
    worst = 0
    for w in _WORKSPACES.values():
        torch.cuda.synchronize(w.buf.device)
        worst = max(worst, int(w.buf[4:8].view(torch.int32).item()))
    return worst


def clear_workspace_cache() -> None:
    """Drop the cached per-stream workspaces (frees their device memory once the
    work queued on them is complete) and the per-signature call plans."""
    _WORKSPACES.clear()
    _TLS.__dict__.pop("plans", None)


def _check_inputs(q: Tensor, k: Tensor, v: Tensor, attn_mask, T: int, B: int) -> None:
    for name, t in (("q", q), ("k", k), ("v", v)):
        if not isinstance(t, torch.Tensor):
            raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
        if t.dim() != 4:
            raise ValueError(f"{name} must have shape (E, H, N, D), got {tuple(t.shape)}")
    if q.shape != k.shape:
        raise ValueError(f"q and k must have the same shape, got {tuple(q.shape)} and {tuple(k.shape)}")
    if v.shape[:3] != q.shape[:3]:
        raise ValueError(f"v must share (E, H, N) with q, got {tuple(v.shape)} vs {tuple(q.shape)}")
    if q.dtype != k.dtype:
        raise TypeError(f"q and k must have the same dtype, got {q.dtype} and {k.dtype}")
    if q.dtype not in _DTYPES or v.dtype not in _DTYPES:
        raise TypeError(f"supported dtypes are float32, float16, bfloat16; got q {q.dtype}, v {v.dtype}")
    if not (q.device == k.device == v.device):
        raise ValueError("q, k and v must be on the same device")
    if min(q.shape) < 1 or v.shape[-1] < 1:
        raise ValueError(f"empty tensors are not supported, got q {tuple(q.shape)}, v {tuple(v.shape)}")
    if not isinstance(B, int) or B < 1:
        raise ValueError(f"block size B must be a positive int, got {B!r}")
    if not isinstance(T, int) or T < 1:
        raise ValueError(f"number of steps T must be a positive int, got {T!r}")
    if attn_mask is not None:
        if attn_mask.shape != (q.shape[0], q.shape[2]):
            raise ValueError(f"attn_mask must have shape (E, N) = {(q.shape[0], q.shape[2])}, "
                             f"got {tuple(attn_mask.shape)}")
        if attn_mask.device != q.device:
            raise ValueError("attn_mask must be on the same device as q")
    if q.device.type != "cuda":
        raise ValueError(f"the 'hip' implementation needs tensors on a GPU, got {q.device}")


def _inner_contiguous(t: Tensor) -> Tensor:
    """The library wants unit stride along the last dimension and token rows that do not overlap
    (stride(2) >= row width); batch and head dimensions may be broadcast.  Anything else - e.g. an
    expand() along the tokens - is copied once."""
    if not (t.stride(-1) == 1 or t.shape[-1] == 1):
        return t.contiguous()
    if t.shape[2] > 1 and t.stride(2) < t.shape[-1]:
        return t.contiguous()
    return t


def _empty_like_layout(v: Tensor, shape) -> Tensor:
    """Output buffer in v's memory layout: models pass (E,H,N,D) views of
    (E,N,H,D) projections (experiments/vit/model.py:73-79) and turn the result
    back with ``permute(0, 2, 1, 3).contiguous()`` (:99) - with the output backed
    by an (E,N,H,Dv) buffer that copy is a no-op.  Anything else gets a
    contiguous (E,H,N,Dv) tensor."""
    E, H, N, Dv = shape
    if H > 1 and N > 1 and v.permute(0, 2, 1, 3).is_contiguous() and not v.is_contiguous():
        return torch.empty((E, N, H, Dv), dtype=v.dtype, device=v.device).permute(0, 2, 1, 3)
    return torch.empty(shape, dtype=v.dtype, device=v.device)


def make_params(q: Tensor, k: Tensor, v: Tensor, mask_u8, out: Tensor, T: int, B: int, pre_pad: bool,
                variant: str = "auto", eps: float = 1e-12) -> L.FwdParams:
    """Fill a ``ma_fwd_params`` (workspace fields left empty)."""
    if variant not in L.VARIANTS:
        raise ValueError(f"unknown variant {variant!r}; available: {', '.join(L.VARIANTS)}")
    E, H, N, D = q.shape
    p = L.FwdParams()
    p.q, p.k, p.v, p.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    p.mask = mask_u8.data_ptr() if mask_u8 is not None else None
    p.mask_dtype = _MASK_DTYPES[mask_u8.dtype] if mask_u8 is not None else L.MA_MASK_U8
    p.E, p.H, p.N, p.D, p.Dv = E, H, N, D, v.shape[-1]
    p.B, p.T, p.pre_pad = B, T, int(bool(pre_pad))
    p.dtype_qk, p.dtype_v = _DTYPES[q.dtype], _DTYPES[v.dtype]
    p.variant = L.VARIANTS[variant]
    for name, t in (("q_stride", q), ("k_stride", k), ("v_stride", v), ("out_stride", out)):
        s = t.stride()
        setattr(p, name, (L.C.c_int64 * 3)(s[0], s[1], s[2]))
    if mask_u8 is not None:
        p.mask_stride = (L.C.c_int64 * 2)(*mask_u8.stride())
    p.eps = eps
    return p


# Filling a ma_fwd_params field by field, validating the arguments and asking the library for the
# workspace size cost more host time than a small forward takes on the GPU, and a model calls the
# operator with the same few signatures over and over.  Everything that depends on the signature
# alone - shapes, strides, dtypes, devices, pointer alignment, T, B, padding side, variant - is
# worked out once and kept as a plan: a validated, filled parameter block that later calls only
# patch pointers into.  Plans are per thread (a block is modified in place right before the call).
_TLS = threading.local()
_PLAN_MAX = 256


class _Plan:
    __slots__ = ("p", "ref", "nbytes", "syncing", "flags", "permuted", "alloc_shape", "dtype", "device", "index")


def _signature(q: Tensor, k: Tensor, v: Tensor, attn_mask, T, B, pre_pad, variant, align: int) -> tuple:
    return (q.shape, k.shape, v.shape, q.stride(), k.stride(), v.stride(), q.dtype, k.dtype, v.dtype,
            q.device, k.device, v.device, T, B, not pre_pad, variant, DEVICE_EXCLUSIVE, _TEST_FLAGS, align,
            None if attn_mask is None else (attn_mask.shape, attn_mask.stride(), attn_mask.dtype, attn_mask.device))


def _make_plan(lib, q: Tensor, k: Tensor, v: Tensor, attn_mask, T: int, B: int, pre_pad, variant):
    """Validate a call signature and prepare its parameter block; None for inputs that have to be
    copied first (the general path does that)."""
    _check_inputs(q, k, v, attn_mask, T, B)
    if _inner_contiguous(q) is not q or _inner_contiguous(k) is not k or _inner_contiguous(v) is not v:
        return None
    mask_u8 = _mask_bytes(attn_mask)
    E, H, N, _ = q.shape
    plan = _Plan()
    with torch.cuda.device(q.device):
        out = _empty_like_layout(v, (E, H, N, v.shape[-1]))
    plan.permuted = not out.is_contiguous()
    plan.alloc_shape = (E, N, H, v.shape[-1]) if plan.permuted else (E, H, N, v.shape[-1])
    plan.dtype, plan.device = v.dtype, v.device
    plan.index = v.device.index if v.device.index is not None else torch.cuda.current_device()
    plan.flags = _TEST_FLAGS | (L.MA_FLAG_DEVICE_EXCLUSIVE if DEVICE_EXCLUSIVE else 0)
    p = make_params(q, k, v, mask_u8, out, T, B, pre_pad, variant or DEFAULT_VARIANT)
    p.flags = plan.flags
    plan.nbytes = lib.ma_fwd_workspace_bytes(p)
    if plan.nbytes == 0:   # invalid problem: let the library say why
        L.check(lib.ma_fwd_workspace_layout(p, L.WsLayout()), "monarch_attention_hip")
    plan.syncing = lib.ma_fwd_select_variant(p) in _SYNCING
    plan.p, plan.ref = p, L.C.byref(p)
    return plan


def _raw_stream(index: int) -> int:
    return torch._C._cuda_getCurrentRawStream(index)


def monarch_attention_hip(q: Tensor, k: Tensor, v: Tensor, attn_mask: Tensor | None, T: int, B: int,
                          pre_pad: bool, *, variant: str | None = None) -> Tensor:
    """MonarchAttention forward on the current HIP stream; returns a new
    ``(E, H, N, Dv)`` tensor of ``v.dtype`` in v's memory layout (contiguous for
    contiguous v; backed by ``(E, N, H, Dv)`` when v is such a permuted view).
    Differentiable with respect to q, k and v: when one of them requires grad
    (and grad mode is on) the call is recorded as one autograd node whose
    backward is ``ma_bwd``."""
    try:
        needs_grad = (q.requires_grad or k.requires_grad or v.requires_grad) and torch.is_grad_enabled()
        qp, kp, vp = q.data_ptr(), k.data_ptr(), v.data_ptr()
        key = _signature(q, k, v, attn_mask, T, B, pre_pad, variant, (qp | kp | vp) & 15)
    except (AttributeError, TypeError):
        _check_inputs(q, k, v, attn_mask, T, B)   # says what is wrong with the arguments
        raise
    if needs_grad:
        _check_inputs(q, k, v, attn_mask, T, B)
        return _MonarchAttentionHip.apply(q, k, v, attn_mask, T, B, bool(pre_pad), variant)
    try:
        plans = _TLS.plans
    except AttributeError:
        plans = _TLS.plans = {}
    plan = plans.get(key, False)
    if plan is False:
        plan = _make_plan(L.load(), q, k, v, attn_mask, T, B, pre_pad, variant)
        if len(plans) >= _PLAN_MAX:
            plans.clear()
        plans[key] = plan
    if plan is None or torch.cuda.current_device() != plan.index:
        return _forward(q, k, v, attn_mask, T, B, pre_pad, variant)
    out = torch.empty(plan.alloc_shape, dtype=plan.dtype, device=plan.device)
    if plan.permuted:
        out = out.permute(0, 2, 1, 3)
    stream = _raw_stream(plan.index)
    w = _WORKSPACES.get((plan.index, stream))
    if w is None or w.nbytes < plan.nbytes:
        w = _workspace(plan.device, stream, plan.nbytes)
    if w.err[0]:
        _raise_failed(w)   # an earlier call on this workspace failed
    p = plan.p
    p.q, p.k, p.v, p.out = qp, kp, vp, out.data_ptr()
    if attn_mask is not None:
        p.mask = attn_mask.data_ptr()
    p.workspace, p.workspace_bytes, p.error_word = w.ptr, w.nbytes, w.err_ptr
    p.flags = plan.flags if w.dirty else plan.flags | L.MA_FLAG_SYNC_READY
    st = _FWD(plan.ref, stream)
    if st:
        L.check(st, "ma_fwd")
    if plan.syncing:
        w.dirty = False   # the library cleared the sync area in front of this launch if it had to
    return out


def _FWD(ref, stream) -> int:
    """ma_fwd of the loaded library (replaces itself by the bound function on first use)."""
    global _FWD
    _FWD = L.load().ma_fwd
    return _FWD(ref, stream)


def _forward(q: Tensor, k: Tensor, v: Tensor, attn_mask, T: int, B: int, pre_pad: bool, variant) -> Tensor:
    """The general path: any device, inputs that need a copy first; nothing is cached."""
    lib = L.load()
    _check_inputs(q, k, v, attn_mask, T, B)
    q, k, v = _inner_contiguous(q), _inner_contiguous(k), _inner_contiguous(v)
    mask_u8 = _mask_bytes(attn_mask)
    E, H, N, _ = q.shape
    with torch.cuda.device(q.device):
        out = _empty_like_layout(v, (E, H, N, v.shape[-1]))
        p = make_params(q, k, v, mask_u8, out, T, B, pre_pad, variant or DEFAULT_VARIANT)
        p.flags = _TEST_FLAGS | (L.MA_FLAG_DEVICE_EXCLUSIVE if DEVICE_EXCLUSIVE else 0)
        nbytes = lib.ma_fwd_workspace_bytes(p)
        if nbytes == 0:   # invalid problem: let the library say why
            L.check(lib.ma_fwd_workspace_layout(p, L.WsLayout()), "monarch_attention_hip")
        syncing = lib.ma_fwd_select_variant(p) in _SYNCING
        stream = torch.cuda.current_stream(q.device).cuda_stream
        w = _workspace(q.device, stream, nbytes)
        if w.err[0]:
            _raise_failed(w)   # an earlier call on this workspace failed
        p.workspace, p.workspace_bytes, p.error_word = w.ptr, w.nbytes, w.err_ptr
        if not w.dirty:
            p.flags |= L.MA_FLAG_SYNC_READY
        L.check(lib.ma_fwd(p, stream), "ma_fwd")
        if syncing:
            w.dirty = False   # the library cleared the sync area in front of this launch if it had to
    return out


def _mask_bytes(attn_mask):
    """The mask as the library reads it: in place, whatever its dtype (bool, any integer, any
    float: non-zero = keep, the truthiness torch.logical_and sees, ma/ma_torch.py:98) and whatever
    its strides.  bool is reinterpreted as bytes; nothing is copied or converted."""
    if attn_mask is None:
        return None
    if attn_mask.dtype == torch.bool:
        return attn_mask.view(torch.uint8)
    if attn_mask.dtype not in _MASK_DTYPES:
        raise TypeError(f"attn_mask dtype {attn_mask.dtype} is not supported")
    return attn_mask


def monarch_matrix_hip(q: Tensor, k: Tensor, attn_mask: Tensor | None, T: int, B: int, pre_pad: bool, *,
                       variant: str | None = None) -> Tensor:
    """Dense ``(E, H, N, N)`` fp32 attention matrix of q and k: what the forward
    pass returns for an fp32 identity as v (``MonarchAttention.get_matrix``,
    ma/monarch_attention.py:61-66), written entry by entry by ``ma_matrix``
    without the identity and without the ``(E, H, Np, N)`` intermediate.
    ``variant`` ('auto', 'generic' or 'staged') selects the kernels of the T
    steps.  Raises ``NotImplementedError`` when the padded sequence is beyond
    what the kernel holds on chip."""
    _check_inputs(q, k, q, attn_mask, T, B)
    lib = L.load()
    q, k = _inner_contiguous(q), _inner_contiguous(k)
    mask_u8 = _mask_bytes(attn_mask)
    E, H, N, _ = q.shape
    with torch.cuda.device(q.device):
        A = torch.empty((E, H, N, N), dtype=torch.float32, device=q.device)
        p = make_params(q, k, q, mask_u8, A, T, B, pre_pad, variant or DEFAULT_VARIANT)
        nbytes = lib.ma_fwd_workspace_bytes(p)
        if nbytes == 0:
            L.check(lib.ma_fwd_workspace_layout(p, L.WsLayout()), "monarch_matrix_hip")
        stream = torch.cuda.current_stream(q.device).cuda_stream
        ws = _workspace(q.device, stream, nbytes).buf
        p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
        p.flags = L.MA_FLAG_SYNC_READY
        st = lib.ma_matrix(p, A.data_ptr(), stream)
        if st == L.MA_ERR_UNSUPPORTED:
            raise NotImplementedError("ma_matrix: " + L.strerror(st))
        L.check(st, "ma_matrix")
    return A


def monarch_attention_hip_backward(q: Tensor, k: Tensor, v: Tensor, attn_mask: Tensor | None, dout: Tensor, T: int,
                                   B: int, pre_pad: bool, *, variant: str | None = None):
    """Gradients ``(dq, dk, dv)`` of ``monarch_attention_hip(q, k, v, attn_mask, T, B, pre_pad)``
    for the output gradient ``dout`` - what autograd through the reference's
    ``monarch_attention_torch`` (ma/ma_torch.py:65-108) yields.  ``ma_bwd`` runs
    the T steps again (``variant`` 'auto', 'generic' or 'staged' picks their
    kernels) and then the backward kernels, all on the current stream."""
    _check_inputs(q, k, v, attn_mask, T, B)
    if dout.shape != v.shape or dout.device != v.device:
        raise ValueError(f"dout must have the shape of the output {tuple(v.shape)}, got {tuple(dout.shape)}")
    lib = L.load()
    q, k, v = _inner_contiguous(q), _inner_contiguous(k), _inner_contiguous(v)
    dout = _inner_contiguous(dout.to(v.dtype))
    mask_u8 = _mask_bytes(attn_mask)
    with torch.cuda.device(q.device):
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        b = L.BwdParams()
        b.fwd = make_params(q, k, v, mask_u8, dv, T, B, pre_pad, variant or DEFAULT_VARIANT)
        b.dout, b.dq, b.dk, b.dv = dout.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
        for name, t in (("dout_stride", dout), ("dq_stride", dq), ("dk_stride", dk), ("dv_stride", dv)):
            setattr(b, name, (L.C.c_int64 * 3)(*t.stride()[:3]))
        nbytes = lib.ma_bwd_workspace_bytes(b)
        if nbytes == 0:
            L.check(lib.ma_fwd_workspace_layout(b.fwd, L.WsLayout()), "monarch_attention_hip_backward")
            raise NotImplementedError("ma_bwd does not support this problem (variant or block shape)")
        stream = torch.cuda.current_stream(q.device).cuda_stream
        # the backward workspace holds every step's state: allocated per call and freed after it
        ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
        b.fwd.workspace, b.fwd.workspace_bytes = ws.data_ptr(), ws.numel()
        L.check(lib.ma_bwd(b, stream), "ma_bwd")
    return dq, dk, dv


class _MonarchAttentionHip(torch.autograd.Function):
    """One autograd node per operator call: forward ``ma_fwd``, backward ``ma_bwd``."""

    @staticmethod
    def forward(ctx, q, k, v, attn_mask, T, B, pre_pad, variant):
        ctx.save_for_backward(q, k, v, attn_mask)
        ctx.args = (T, B, pre_pad, variant if variant in ("auto", "generic", "staged") else None)
        return _forward(q, k, v, attn_mask, T, B, pre_pad, variant)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dout):
        q, k, v, attn_mask = ctx.saved_tensors
        T, B, pre_pad, variant = ctx.args
        dq, dk, dv = monarch_attention_hip_backward(q, k, v, attn_mask, dout, T, B, pre_pad, variant=variant)
        return dq, dk, dv, None, None, None, None, None
