"""``torch.ops.lvar.*``: the three attention ops with the schemas the reference registers as
``torch.ops.chipmunk.*`` (kernels/chipmunk/csrc/chipmunk.cu:57-59), for callers that use the
torch-library entry points directly (``SelfAttention.forward`` calls ``torch.ops.chipmunk.dense_attn``,
models/sparvar/basic_sparvar.py:384).  Like the reference's CUDA ops the softmax scale is fixed to 1
(Infinity's cosine attention, dense_attn.cu:161-163); ``lse`` / ``p`` / ``l`` are the reference's
per-row constant ``1 / (2^M * L)`` with the 1 = e^0 scale folded in, shape ``[B,H,Lq,1]``.

    import lvar_amd.torch_ops          # registers the ops
    o, lse = torch.ops.lvar.dense_attn(q, k, v)
    o, cs, l = torch.ops.lvar.dense_colsum_attn(q, k, v, lse)
    torch.ops.lvar.csp_attn(q, k, v, o, indices, counts, -1)      # in place on o
"""
from __future__ import annotations

import torch

from . import _lib
from . import sparse_attn_ops as ops
from .sparse_attn_config import get_kernel_config_attn

_lib_def = torch.library.Library("lvar", "DEF")
_lib_def.define("csp_attn(Tensor q, Tensor k, Tensor v, Tensor(a!) o, Tensor indices, Tensor indices_counts, int o_scale) -> ()")
_lib_def.define("dense_attn(Tensor q, Tensor k, Tensor v) -> Tensor[]")
_lib_def.define("dense_colsum_attn(Tensor q, Tensor k, Tensor v, Tensor p) -> Tensor[]")


def _dense_attn(q, k, v):
    q, k, v = ops._prep(q, "q"), ops._prep(k, "k"), ops._prep(v, "v")
    ops._check_qkv(q, k, v)
    o, _, _, lse2 = ops._dense_launch(q, k, v, 1.0, want_ml=False, want_lse2=True)
    return [o, torch.exp2(-lse2).unsqueeze(-1)]


def _dense_colsum_attn(q, k, v, p):
    q, k, v = ops._prep(q, "q"), ops._prep(k, "k"), ops._prep(v, "v")
    ops._check_qkv(q, k, v)
    if tuple(p.shape) != (q.shape[0], q.shape[1], q.shape[2], 1):
        raise ops.ShapeError(f"P shape mismatch - p: {tuple(p.shape)}, q: {tuple(q.shape)}")
    o, _, _, lse2 = ops._dense_launch(q, k, v, 1.0, want_ml=False, want_lse2=True)
    prev = (-torch.log2(p.to(torch.float32))).reshape(q.shape[:3]).contiguous()
    cs = ops._colsum_given_lse(q, k, prev, 1.0, get_kernel_config_attn()["bm"])
    return [o, cs, torch.exp2(-lse2).unsqueeze(-1)]


def _csp_attn(q, k, v, o, indices, indices_counts, o_scale):
    if o_scale not in (1, -1):
        raise ValueError("o_scale must be 1 or -1")          # csp_attn.cu:330
    qq, kk, vv = ops._prep(q, "q"), ops._prep(k, "k"), ops._prep(v, "v")
    ops._check_qkv(qq, kk, vv)
    if o.dtype != torch.bfloat16 or o.stride(-1) != 1 or tuple(o.shape) != tuple(q.shape):
        raise ops.ShapeError("o must be a bf16 tensor shaped like q with unit stride on the head dimension")
    B, H, Lq, d = qq.shape
    G = indices.shape[2]
    bm = get_kernel_config_attn()["bm"]
    indices = indices.contiguous() if indices.stride(3) != 1 else indices
    counts = indices_counts.contiguous()
    with torch.cuda.device(qq.device):
        st = _lib.load().lvar_csp_attn_fwd(ops._view(qq), ops._view(kk), ops._view(vv), ops._view(o), ops._view(o), None, None,
                                          indices.data_ptr(), counts.data_ptr(), G, indices.stride(2), bm,
                                          B, H, Lq, kk.shape[2], d, float(o_scale), 1.0, ops._stream(qq))
    _lib.check(st, "lvar_csp_attn_fwd")


_lib_impl = torch.library.Library("lvar", "IMPL", "CUDA")
_lib_impl.impl("dense_attn", _dense_attn)
_lib_impl.impl("dense_colsum_attn", _dense_colsum_attn)
_lib_impl.impl("csp_attn", _csp_attn)
