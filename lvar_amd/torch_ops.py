"""Torch-library registration of the three attention ops and the two list-building ops with the schemas the reference
registers as ``torch.ops.chipmunk.*`` (kernels/chipmunk/csrc/chipmunk.cu:57-59, 66-68), for callers that use the
torch-library entry points directly (``SelfAttention.forward`` calls ``torch.ops.chipmunk.dense_attn``,
models/sparvar/basic_sparvar.py:384).  Like the reference's CUDA ops the softmax scale is fixed to 1
(Infinity's cosine attention, dense_attn.cu:161-163); ``lse`` / ``p`` / ``l`` are the reference's
per-row constant ``1 / (2^M * L)`` with the 1 = e^0 scale folded in, shape ``[B,H,Lq,1]``.

    import lvar_amd.torch_ops          # registers torch.ops.lvar.*
    o, lse = torch.ops.lvar.dense_attn(q, k, v)
    o, cs, l = torch.ops.lvar.dense_colsum_attn(q, k, v, lse)
    torch.ops.lvar.csp_attn(q, k, v, o, indices, counts, -1)      # in place on o
    indices, counts = torch.ops.lvar.mask_to_indices(mask, 64, 192)
    torch.ops.lvar.topk_indices(activation, indices, counts, 0.8, 64, 0.0)   # in place on indices / counts

    lvar_amd.torch_ops.register_as("chipmunk")    # opt-in: the reference's call sites then run unedited

``dense_attn`` is implemented natively (checks, allocation and launch in C++, ``csrc/torch_binding.cpp``)
when the compiled binding is built; the other two ops run at shapes where the kernel, not the host, is
the bound and are Python implementations over the same C ABI.  Differences from the reference's CUDA ops:
``cs`` is fp32 ``[B,H,ceil(Lq/192),Lk]`` without row padding (the reference returns bf16 with the row
stride padded to a multiple of 8), and head_dim may be 64 as well as 128.
"""
from __future__ import annotations

import torch

from . import _lib
from . import sparse_attn_ops as ops
from .sparse_attn_config import get_kernel_config_attn

_SCHEMAS = {
    "csp_attn": "csp_attn(Tensor q, Tensor k, Tensor v, Tensor(a!) o, Tensor indices, Tensor indices_counts, int o_scale) -> ()",
    "dense_attn": "dense_attn(Tensor q, Tensor k, Tensor v) -> Tensor[]",
    "dense_colsum_attn": "dense_colsum_attn(Tensor q, Tensor k, Tensor v, Tensor p) -> Tensor[]",
    # indexed IO (chipmunk.cu:66-68)
    "topk_indices": "topk_indices(Tensor activation, Tensor(indices!) indices, Tensor counts, float sparsity_amount, int multiple_of, float random_amount) -> ()",
    "mask_to_indices": "mask_to_indices(Tensor mask, int multiple_of, int pad_to_multiple_of) -> Tensor[]",
}
_registered = {}      # namespace -> the torch.library.Library objects that keep the registration alive


def _dense_attn(q, k, v):
    q, k, v = ops._prep(q, "q"), ops._prep(k, "k"), ops._prep(v, "v")
    ops._check_qkv(q, k, v, gqa=True)
    B, H, Lq, d = q.shape
    o = torch.empty_like(q)
    rcp = torch.empty((B, H, Lq, 1), dtype=torch.float32, device=q.device)
    with ops._on_device(q):
        st = _lib.load().lvar_dense_attn_rcp_fwd(ops._view(q), ops._view(k), ops._view(v), ops._view(o), rcp.data_ptr(),
                                                B, H, k.shape[1], Lq, k.shape[2], d, 1.0, ops._stream(q))
    _lib.check(st, "lvar_dense_attn_rcp_fwd")
    return [o, rcp]


def _dense_colsum_attn(q, k, v, p):
    q, k, v = ops._prep(q, "q"), ops._prep(k, "k"), ops._prep(v, "v")
    ops._check_qkv(q, k, v, gqa=True)                    # dense_colsum_attn.cu:386-387
    if tuple(p.shape) != (q.shape[0], q.shape[1], q.shape[2], 1):
        raise ops.ShapeError(f"P shape mismatch - p: {tuple(p.shape)}, q: {tuple(q.shape)}")
    o, _, _, lse2 = ops._dense_launch(q, k, v, 1.0, want_ml=False, want_lse2=True)
    prev = (-torch.log2(p.to(torch.float32))).reshape(q.shape[:3]).contiguous()
    cs = ops._colsum_given_lse(q, k, prev, 1.0, get_kernel_config_attn()["bm"])
    return [o, cs, torch.exp2(-lse2).unsqueeze(-1)]


def _csp_attn(q, k, v, o, indices, indices_counts, o_scale):
    if o_scale not in (1, -1):
        raise ValueError("o_scale must be 1 or -1")          # csp_attn.cu:330
    if o.dtype != torch.bfloat16 or o.stride(-1) != 1 or tuple(o.shape) != tuple(q.shape) or o.device != q.device \
            or any(s % 8 for s in o.stride()[:-1]) or o.data_ptr() % 16:
        raise ops.ShapeError("o must be a 16-byte aligned bf16 tensor shaped like q, on q's device, with unit stride on the "
                             "head dimension and strides that are multiples of 8")
    # same list checks as the operator-level csp_attn (dtype, dims, counts shape, device, packed (b,h,g) strides);
    # the result is accumulated in place: o is both the addend and the destination
    ops._csp_launch(q, k, v, indices, indices_counts, o, o_scale, 1.0, False, out=o)


def _topk_indices(activation, indices, counts, sparsity_amount, multiple_of, random_amount):
    ops.topk_indices(activation, indices, counts, sparsity_amount, multiple_of, random_amount)


def _mask_to_indices(mask, multiple_of, pad_to_multiple_of):
    return ops.mask_to_indices(mask, multiple_of, pad_to_multiple_of)


_IMPLS = {"dense_attn": _dense_attn, "dense_colsum_attn": _dense_colsum_attn, "csp_attn": _csp_attn,
          "topk_indices": _topk_indices, "mask_to_indices": _mask_to_indices}


def register_as(namespace: str) -> None:
    """Registers the ops under ``torch.ops.<namespace>`` (idempotent).  ``register_as("chipmunk")`` makes
    the reference's call sites (``torch.ops.chipmunk.dense_attn`` at basic_sparvar.py:384, the ``cuda`` provider
    branches of sparse_attn_ops.py:55,84,96,289) resolve to this library; it refuses to do so when another
    extension has already registered one of these ops under that name."""
    if namespace in _registered:
        return
    ns = getattr(torch.ops, namespace)
    taken = [name for name in _SCHEMAS if hasattr(ns, name)]
    if taken:
        raise RuntimeError(f"torch.ops.{namespace} already has {taken}: another extension owns these ops")
    keep = []
    native = _lib.torch_binding()
    frag = torch.library.Library(namespace, "FRAGMENT")
    for name, schema in _SCHEMAS.items():
        if name == "dense_attn" and native is not None:
            native.register_dense_attn(namespace)          # defined and implemented in C++
            continue
        frag.define(schema)
        frag.impl(name, _IMPLS[name], "CUDA")
    keep.append(frag)
    _registered[namespace] = keep


register_as("lvar")
