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

# One workspace per (device, stream), grown on demand and reused call after
# call: calls on one stream are ordered, so they can share it.  It is allocated
# zero-filled, and every forward call leaves its sync area in the state the next
# call needs (counters and epochs continuing), which is what
# MA_FLAG_SYNC_READY promises to the library.
#
# The one-launch kernels (fused, chained) wait for each other's workgroups with
# bounded waits; a wait that runs out raises a sticky error word in the
# workspace and the workgroup writes NaN instead of results.  That word is
# brought to the host WITHOUT synchronising: every few calls a 4-byte copy into
# pinned memory is queued on a side stream behind the forward kernel, and the
# next call on the workspace that finds the copy complete looks at it - a failed
# call is reported by a RuntimeError from a later call, the sync area is cleared
# again, and the call after that is a normal one.
_CHECK_EVERY = 16          # calls between two looks at the error word (the first call always looks)
_TEST_FLAGS = 0            # extra ma_fwd_params.flags for the failure-path tests (MA_FLAG_TEST_NO_SPIN)
_SYNCING = (L.VARIANTS["fused"], L.VARIANTS["chained"])


class _Workspace:
    def __init__(self, device: torch.device, nbytes: int):
        self.buf = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        self.err_host = torch.zeros(1, dtype=torch.int32, pin_memory=True)
        self.pending = None     # (event on the side stream, buffer the copy reads from)
        self.calls = 0
        self.dirty = False      # the sync area must be cleared before the next one-launch kernel


_WORKSPACES: dict[tuple[int, int], _Workspace] = {}
_SIDE_STREAMS: dict[int, torch.cuda.Stream] = {}


def _workspace(device: torch.device, stream_ptr: int, nbytes: int) -> _Workspace:
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_ptr)
    w = _WORKSPACES.get(key)
    if w is None:
        w = _WORKSPACES[key] = _Workspace(device, nbytes)
    elif w.buf.numel() < nbytes:
        if w.pending is not None:          # let the queued look at the old buffer finish first
            w.pending[0].synchronize()
            _collect(w)
        w.buf = torch.zeros(nbytes, dtype=torch.uint8, device=device)
    return w


def _collect(w: _Workspace) -> None:
    """Look at a completed copy of the error word; raise if a call on this workspace failed."""
    w.pending = None
    code = int(w.err_host.item())
    if code == 0:
        return
    w.err_host.zero_()
    w.dirty = True
    w.buf[4:8].zero_()      # the word is sticky: clear it for the calls to come
    what = {1: "a bounded wait between workgroups ran out",
            2: "workgroups of one head ran on different XCDs (the one-launch kernels rely on ids x, x + 8, ... "
               "sharing an XCD)"}.get(code, f"error word {code}")
    raise RuntimeError(f"monarch_attention_hip: an earlier forward call on this stream failed: {what}; its output "
                       f"holds NaN rows.  The workspace has been reset; pass variant='staged' to avoid the "
                       f"one-launch kernels")


def _queue_check(w: _Workspace, device: torch.device, main: "torch.cuda.Stream") -> None:
    """Queue a copy of the error word to pinned memory behind the work queued on `main` so far,
    on a side stream: the main stream never waits for it."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    side = _SIDE_STREAMS.get(idx)
    if side is None:
        side = _SIDE_STREAMS[idx] = torch.cuda.Stream(device=device)
    after = torch.cuda.Event()
    after.record(main)
    side.wait_event(after)
    with torch.cuda.stream(side):
        w.err_host.copy_(w.buf[4:8].view(torch.int32), non_blocking=True)
        done = torch.cuda.Event()
        done.record(side)
    w.pending = (done, w.buf)


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
    """Drop the cached per-stream workspaces (frees their device memory)."""
    for w in _WORKSPACES.values():
        if w.pending is not None:
            w.pending[0].synchronize()
    _WORKSPACES.clear()


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


# Filling a ma_fwd_params field by field costs more host time than a small forward takes on the
# GPU, and a model calls the operator with the same few shapes over and over: the filled block
# (and the workspace size the library reports for it) is kept per call signature, and a call only
# copies it and patches the pointers.
_PARAM_CACHE: dict[tuple, tuple] = {}
_PARAM_CACHE_MAX = 256


def _params_for(lib, q: Tensor, k: Tensor, v: Tensor, mask_u8, out: Tensor, T: int, B: int, pre_pad: bool,
                variant: str) -> tuple:
    key = (q.shape, q.stride(), k.stride(), v.shape, v.stride(), out.stride(),
           None if mask_u8 is None else (mask_u8.stride(), mask_u8.dtype), q.dtype, v.dtype, T, B, bool(pre_pad), variant)
    hit = _PARAM_CACHE.get(key)
    if hit is None:
        tmpl = make_params(q, k, v, mask_u8, out, T, B, pre_pad, variant)
        nbytes = lib.ma_fwd_workspace_bytes(tmpl)
        if nbytes == 0:   # invalid problem: let the library say why
            L.check(lib.ma_fwd_workspace_layout(tmpl, L.WsLayout()), "monarch_attention_hip")
        if len(_PARAM_CACHE) >= _PARAM_CACHE_MAX:
            _PARAM_CACHE.clear()
        hit = _PARAM_CACHE[key] = (bytes(tmpl), nbytes, lib.ma_fwd_select_variant(tmpl))
    p = L.FwdParams.from_buffer_copy(hit[0])
    p.q, p.k, p.v, p.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    p.mask = mask_u8.data_ptr() if mask_u8 is not None else None
    return p, hit[1], hit[2]


def monarch_attention_hip(q: Tensor, k: Tensor, v: Tensor, attn_mask: Tensor | None, T: int, B: int,
                          pre_pad: bool, *, variant: str | None = None) -> Tensor:
    """MonarchAttention forward on the current HIP stream; returns a new
    ``(E, H, N, Dv)`` tensor of ``v.dtype`` in v's memory layout (contiguous for
    contiguous v; backed by ``(E, N, H, Dv)`` when v is such a permuted view).
    Differentiable with respect to q, k and v: when one of them requires grad
    (and grad mode is on) the call is recorded as one autograd node whose
    backward is ``ma_bwd``."""
    _check_inputs(q, k, v, attn_mask, T, B)
    if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
        return _MonarchAttentionHip.apply(q, k, v, attn_mask, T, B, bool(pre_pad), variant)
    return _forward(q, k, v, attn_mask, T, B, pre_pad, variant)


def _forward(q: Tensor, k: Tensor, v: Tensor, attn_mask, T: int, B: int, pre_pad: bool, variant) -> Tensor:
    lib = L.load()
    q, k, v = _inner_contiguous(q), _inner_contiguous(k), _inner_contiguous(v)
    mask_u8 = _mask_bytes(attn_mask)
    E, H, N, _ = q.shape
    with torch.cuda.device(q.device):
        out = _empty_like_layout(v, (E, H, N, v.shape[-1]))
        p, nbytes, resolved = _params_for(lib, q, k, v, mask_u8, out, T, B, pre_pad, variant or DEFAULT_VARIANT)
        main = torch.cuda.current_stream(q.device)
        w = _workspace(q.device, main.cuda_stream, nbytes)
        if w.pending is not None and w.pending[0].query():
            _collect(w)   # raises if an earlier call on this workspace failed
        p.workspace, p.workspace_bytes = w.buf.data_ptr(), w.buf.numel()
        p.flags = (0 if w.dirty else L.MA_FLAG_SYNC_READY) | _TEST_FLAGS
        L.check(lib.ma_fwd(p, main.cuda_stream), "ma_fwd")
        if resolved in _SYNCING:
            w.dirty = False   # the library cleared the sync area in front of this launch if it had to
            if w.pending is None and (w.calls % _CHECK_EVERY == 0 or _TEST_FLAGS):
                _queue_check(w, q.device, main)
            w.calls += 1
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
