"""Public entry point and ``torch.library`` operator layer of the MI355X implementation.

Drop-in for the reference's ``chill_attention/chill.py``: ``chill_attention(q, k, v, mask=...)``
with the same keyword surface, one ``chill_attention::forward{Mask}`` / ``backward{Mask}`` custom-op
pair per mask class (same argument order), fake (meta) implementations for ``torch.compile`` and
an autograd formula.  Underneath, the adapters allocate outputs with torch and hand raw pointers
and strides to the C ABI of the HIP library; there is no other compute path.
"""

from __future__ import annotations

import ctypes
import logging
import math
import typing

import torch
import torch.nn.functional as F

from . import _lib
from .mask import ChillMask, _descriptor

logger = logging.getLogger(__name__)

_DTYPES = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}
_HEAD_DIMS = (16, 32, 64, 128, 256)


def _kernel_view(t: torch.Tensor) -> torch.Tensor:
    """A view the kernels can address (unit inner stride, 16-byte aligned rows), copying only if
    the tensor does not already qualify."""
    es = t.element_size()
    ok = (
        t.stride(-1) == 1
        and t.data_ptr() % 16 == 0
        and all(s >= 0 and (s * es) % 16 == 0 for s in t.stride()[:-1])
    )
    return t if ok else t.contiguous()


def _stream_ptr(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _require(cond: bool, message: str):
    # explicit raises: input validation must survive ``python -O``
    if not cond:
        raise ValueError(f"chill_attention: {message}")


def _check_inputs(q, k, v, lens, sm_scale, others=()):
    """Shapes, dtypes and devices of one call; ``others`` = further tensors (o, lse, do) that must live
    on q's device.  Everything the kernels dereference is checked here: a tensor on the CPU or on
    another GPU would reach them as a bad pointer."""
    _require(q.ndim == 4 and k.ndim == 4 and v.ndim == 4, "q, k, v must be [B, H, T, D]")
    batch, heads, T, head_dim = q.shape
    num_kv_heads = k.shape[1]
    _require(heads % num_kv_heads == 0, "the number of query heads must be a multiple of the key/value heads")
    _require(head_dim in _HEAD_DIMS, f"head dim must be one of {_HEAD_DIMS}")
    _require(head_dim == k.shape[-1] and head_dim == v.shape[-1], "q, k, v must share the head dim")
    _require(T == k.shape[-2] and T == v.shape[-2], "q, k, v must share the sequence length")
    _require(k.shape[0] == batch and v.shape[0] == batch and v.shape[1] == num_kv_heads, "batch / head mismatch")
    _require(q.dtype in _DTYPES and k.dtype == q.dtype and v.dtype == q.dtype, "q, k, v must share a dtype of fp32 / fp16 / bf16")
    _require(sm_scale is not None and math.isfinite(float(sm_scale)), "sm_scale must be a finite number")
    _require(lens is None or (lens.dtype == torch.int32 and lens.ndim == 1 and batch == len(lens)),
             "lens must be an int32 vector with one entry per batch element")
    for name, t in (("k", k), ("v", v), ("lens", lens)) + tuple(others):
        _require(t is None or t.device == q.device, f"{name} is on {t.device if t is not None else None}, q on {q.device}")
    if not q.is_cuda:
        raise RuntimeError("chill_attention runs on the GPU only (tensors must be on a ROCm 'cuda' device)")


def _lens_args(lens: typing.Optional[torch.Tensor]):
    if lens is None:
        return None, 0
    return ctypes.c_void_p(lens.data_ptr()), lens.stride(0)


def register_chill_mask(mask: ChillMask):
    """Register the forward / backward custom ops of ``mask``'s class (once per class name).

    Instances of one class share the ops; their ``constargs`` travel as the ``mask_args``
    operand and reach the kernels as run-time values.
    """
    mask_name = mask.name
    if hasattr(torch.ops.chill_attention, f"forward{mask_name}"):
        return
    mask_cls = type(mask)

    # the library that holds this class's functor (a user-written mask has one of its own, built
    # here on first registration)
    mask_lib = mask_cls._library()

    def mask_cls_descriptor(mask_args):
        return _descriptor(mask_cls, tuple(mask_args))

    @torch.library.custom_op(
        f"chill_attention::forward{mask_name}", mutates_args=(), device_types=("cuda",)
    )
    def attention_forward_adapter(
        q: torch.Tensor,
        k: torch.Tensor,
        v: torch.Tensor,
        lens: typing.Optional[torch.Tensor],
        mask_args: typing.List[typing.Union[int, float, bool]],
        sm_scale: float,
        return_lse: bool,
        prescale_qk: bool,
        precision: str,
        autotune: bool,
    ) -> tuple[torch.Tensor, torch.Tensor]:
        _check_inputs(q, k, v, lens, sm_scale)
        batch, heads, T, head_dim = q.shape
        desc = mask_cls_descriptor(mask_args)
        qv, kv, vv = _kernel_view(q), _kernel_view(k), _kernel_view(v)
        # the kernel writes every row (zeros where nothing attends), so no zero fill is needed
        O = torch.empty_like(q, memory_format=torch.contiguous_format)
        LSE = None
        if return_lse:
            LSE = torch.empty(q.shape[:3], dtype=torch.float32, device=q.device)
        lens_ptr, lens_stride = _lens_args(lens)
        tq, tk, tv, to = _lib.tensor4(qv), _lib.tensor4(kv), _lib.tensor4(vv), _lib.tensor4(O)
        with torch.cuda.device(q.device):
            status = mask_lib.chill_fwd(
                ctypes.byref(tq), ctypes.byref(tk), ctypes.byref(tv), ctypes.byref(to),
                ctypes.c_void_p(LSE.data_ptr()) if LSE is not None else None,
                _lib.strides3(LSE) if LSE is not None else None,
                lens_ptr, lens_stride,
                batch, heads, k.shape[1], T, head_dim, _DTYPES[q.dtype], float(sm_scale),
                ctypes.byref(desc), ctypes.c_void_p(_stream_ptr(q)),
            )
        _lib.check("chill_fwd", status)
        if LSE is None:
            LSE = torch.empty(0, device=q.device)
        return O, LSE

    @torch.library.register_fake(f"chill_attention::forward{mask_name}")
    def attention_forward_adapter_abstract(
        q, k, v, lens, mask_args, sm_scale, return_lse, prescale_qk, precision, autotune
    ):
        return (
            torch.empty_like(q, memory_format=torch.contiguous_format),
            torch.empty(q.shape[:3], dtype=torch.float32, device=q.device)
            if return_lse
            else torch.empty(0, device=q.device),
        )

    @torch.library.custom_op(
        f"chill_attention::backward{mask_name}", mutates_args=(), device_types=("cuda",)
    )
    def attention_backward_adapter(
        q: torch.Tensor,
        k: torch.Tensor,
        v: torch.Tensor,
        lens: typing.Optional[torch.Tensor],
        o: torch.Tensor,
        lse: torch.Tensor,
        do: torch.Tensor,
        mask_args: typing.List[typing.Union[int, float, bool]],
        sm_scale: float,
        prescale_qk: bool,
        precision: str,
        autotune: bool,
    ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        _check_inputs(q, k, v, lens, sm_scale, others=(("o", o), ("lse", lse), ("do", do)))
        _require(o.shape == q.shape and do.shape == q.shape and lse.shape == q.shape[:3], "o, do, lse must match q")
        batch, heads, T, head_dim = q.shape
        num_kv_heads = k.shape[1]
        desc = mask_cls_descriptor(mask_args)
        dtype = _DTYPES[q.dtype]
        qv, kv, vv, ov = _kernel_view(q), _kernel_view(k), _kernel_view(v), _kernel_view(o)
        dov = _kernel_view(do if do.dtype == q.dtype else do.to(q.dtype))
        lse = lse.contiguous()
        delta = torch.empty(o.shape[:-1], dtype=torch.float32, device=o.device)
        DQ = torch.empty_like(q, memory_format=torch.contiguous_format)
        DK = torch.empty_like(k, memory_format=torch.contiguous_format)
        DV = torch.empty_like(v, memory_format=torch.contiguous_format)
        lens_ptr, lens_stride = _lens_args(lens)
        tq, tk, tv, to, tdo = (_lib.tensor4(x) for x in (qv, kv, vv, ov, dov))
        tdq, tdk, tdv = _lib.tensor4(DQ), _lib.tensor4(DK), _lib.tensor4(DV)
        stream = ctypes.c_void_p(_stream_ptr(q))
        lse_p, delta_p = ctypes.c_void_p(lse.data_ptr()), ctypes.c_void_p(delta.data_ptr())
        with torch.cuda.device(q.device):
            # dQ first: it computes delta = rowsum(O * dO) of its rows on the way (the reference's separate
            # preprocessing launch, chill.py:278-290) and leaves it in `delta` for dK/dV
            _lib.check(
                "chill_bwd_dq_delta",
                mask_lib.chill_bwd_dq_delta(
                    ctypes.byref(tq), ctypes.byref(tk), ctypes.byref(tv), ctypes.byref(to), ctypes.byref(tdo),
                    ctypes.byref(tdq),
                    lse_p, _lib.strides3(lse), delta_p, _lib.strides3(delta), lens_ptr, lens_stride,
                    batch, heads, num_kv_heads, T, head_dim, dtype, float(sm_scale),
                    ctypes.byref(desc), stream,
                ),
            )
            _lib.check(
                "chill_bwd_dkdv",
                mask_lib.chill_bwd_dkdv(
                    ctypes.byref(tq), ctypes.byref(tk), ctypes.byref(tv), ctypes.byref(tdo),
                    ctypes.byref(tdk), ctypes.byref(tdv),
                    lse_p, _lib.strides3(lse), delta_p, _lib.strides3(delta), lens_ptr, lens_stride,
                    batch, heads, num_kv_heads, T, head_dim, dtype, float(sm_scale),
                    ctypes.byref(desc), stream,
                ),
            )
        return DQ, DK, DV

    @torch.library.register_fake(f"chill_attention::backward{mask_name}")
    def attention_backward_adapter_abstract(
        q, k, v, lens, o, lse, do, mask_args, sm_scale, prescale_qk, precision, autotune
    ):
        return (
            torch.empty_like(q, memory_format=torch.contiguous_format),
            torch.empty_like(k, memory_format=torch.contiguous_format),
            torch.empty_like(v, memory_format=torch.contiguous_format),
        )

    def setup_context(ctx, inputs, output):
        O, LSE = output
        q, k, v, lens, mask_args, sm_scale, return_lse, prescale_qk, precision, autotune = inputs
        ctx.save_for_backward(q, k, v, O, LSE, lens)
        ctx.mask_args = mask_args
        ctx.sm_scale = sm_scale
        ctx.prescale_qk = prescale_qk
        ctx.precision = precision
        ctx.autotune = autotune

    def backward(ctx, do, dlse):
        # LSE is not differentiated (as in the reference); one gradient per forward input
        q, k, v, o, lse, lens = ctx.saved_tensors
        DQ, DK, DV = attention_backward_adapter(
            q, k, v, lens, o, lse, do, ctx.mask_args, ctx.sm_scale, ctx.prescale_qk, ctx.precision, ctx.autotune,
        )
        return DQ, DK, DV, None, None, None, None, None, None, None

    attention_forward_adapter.register_autograd(backward, setup_context=setup_context)


def _chill_reference_naive(
    mask: ChillMask,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    lens: typing.Optional[torch.Tensor],
):
    """Dense-mask attention through ``torch`` SDPA, for testing.

    Expands GQA heads, materialises ``mask.make_mask(T)``, restricts keys and queries to
    ``lens`` when given, and returns ``(output * res_mask, res_mask)`` where ``res_mask`` zeroes
    the padded query rows (1 if ``lens`` is None).
    """
    assert q.size(2) == k.size(2)
    if q.shape[1] != k.shape[1]:
        rep = q.shape[1] // k.shape[1]
        k = k.repeat_interleave(rep, dim=1)
        v = v.repeat_interleave(rep, dim=1)
    T = q.size(2)
    attn_mask = mask.make_mask(T).to(q.device)
    res_mask: typing.Any = 1
    if lens is not None:
        in_len = (torch.arange(T, device=q.device)[None, :] < lens[:, None])[:, :, None]  # [B, T, 1]
        pair = in_len & in_len.transpose(-1, -2)  # [B, T, T]
        attn_mask = attn_mask[None, None] & pair[:, None]
        res_mask = in_len[:, None]
    res_mask = torch.as_tensor(res_mask, device=q.device)
    out = F.scaled_dot_product_attention(q, k, v, attn_mask=attn_mask)
    return out * res_mask, res_mask


# mask class -> (C++ operator or None, the operator's handle of the class's kernel library, mask id)
_eager = {}


def _eager_operator(mask: ChillMask):
    cls = type(mask)
    entry = _eager.get(cls)
    if entry is None:
        op = _lib.torch_operator()
        table = mask_id = None
        if op is not None:
            table = _lib.register_entry_points(cls._library())
            mask_id = _descriptor(cls, mask.constargs).id
        entry = _eager[cls] = (op, table, mask_id)
    return entry


def _chill_attention(q, k, v, lens, mask_name, mask_args, sm_scale, return_lse, prescale_qk, precision, autotune):
    requires_grad = any(i.requires_grad for i in (q, k, v))
    forward = getattr(torch.ops.chill_attention, f"forward{mask_name}")
    O, LSE = forward(
        q, k, v, lens, list(mask_args), sm_scale, return_lse or requires_grad, prescale_qk, precision, autotune
    )
    if return_lse:
        return O, LSE
    return O


def chill_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    mask: ChillMask,
    lens: typing.Optional[torch.Tensor] = None,
    sm_scale: typing.Optional[float] = None,
    return_lse=False,
    prescale_qk=False,
    precision="ieee",
    autotune=False,
):
    """Masked flash attention on MI355X.  GQA is active when ``k.shape[1] != q.shape[1]``.

    Args:
        q: ``[B, H, T, D]``; k, v: ``[B, H_kv, T, D]``; fp32, fp16 or bf16, D in {16, 32, 64, 128, 256}.
        mask: a ``ChillMask`` instance.
        lens: optional int32 ``[B]`` valid lengths (values above T are clamped).
        sm_scale: softmax scale, default ``D ** -0.5``.
        return_lse: also return LSE2 ``[B, H, T]`` fp32 (base 2, scale included; ``-inf`` for rows
            that see no key, 0 for rows at or beyond ``lens``).
        prescale_qk, precision, autotune: accepted for interface compatibility.  The scale is
            always applied to the fp32 scores; fp32 inputs always use IEEE fp32 MFMA (gfx950 has no
            tf32 path); tile shapes come from a static table, there is no autotuner.

    Returns:
        ``O`` or ``(O, LSE2)``.
    """
    register_chill_mask(mask)
    if sm_scale is None:
        sm_scale = 1.0 / (q.shape[-1] ** 0.5)
    if not torch.compiler.is_compiling():
        # eager calls take the operator registered from C++ (same adapters, same autograd formula);
        # the torch.library operators below serve torch.compile and builds without that library
        op, table, mask_id = _eager_operator(mask)
        if op is not None:
            _check_inputs(q, k, v, lens, sm_scale)
            mask_args = [int(a) for a in mask.constargs]
            _require(all(a == b for a, b in zip(mask_args, mask.constargs)), "mask arguments must be integers")
            O, LSE = op(q, k, v, lens, table, mask_id, mask_args, float(sm_scale), bool(return_lse))
            return (O, LSE) if return_lse else O
    if not torch.compiler.is_compiling():
        for i in (q, k, v):
            torch._dynamo.mark_static(i, 1)
            torch._dynamo.mark_static(i, 3)
    return _chill_attention(
        q=q, k=k, v=v, lens=lens, mask_name=mask.name, mask_args=mask.constargs, sm_scale=sm_scale,
        return_lse=return_lse, prescale_qk=prescale_qk, precision=precision, autotune=autotune,
    )
