"""CS4A caller: colsum -> top-k key lists -> column-sparse attention with an O-cache.  The counterpart
of the reference's ``SparseDiffAttn._fast_attention`` (models/sparvar/sparse_attn.py:865-1167): same
full-step / sparse-step arithmetic, with the per-layer storage reduced to plain attributes (the
reference's CPU offload pipeline is disabled in its shipped configuration and is not rebuilt)."""
from __future__ import annotations

from typing import Dict, Optional, Sequence, Tuple

import torch

from . import mask_build as mb
from . import sparse_attn_ops as ops
from .sparse_attn_config import GLOBAL_CONFIG, get_kernel_config_attn


class SparseDiffAttn:
    def __init__(self, layer_num: int = 0, use_o_cache: bool = True, scales: Sequence[int] = mb.INFINITY_SCALES,
                 spsd_scale: int = 10, speedup: bool = False):
        self.layer_num = layer_num
        self.use_o_cache = use_o_cache
        self.scales = tuple(scales)
        self.spsd_scale = spsd_scale
        cfg = get_kernel_config_attn()
        self.bm, self.multiple_of, self.indices_pad_to = cfg["bm"], cfg["counts_multiple_of"], cfg["indices_pad_to"]
        ws = list(GLOBAL_CONFIG["attn"]["cs4a_ws"])
        n_sparse = len(self.scales) - (spsd_scale + 1)
        wind = ws[len(ws) - n_sparse:] if n_sparse > 0 else []
        assert len(wind) == n_sparse, "w/ local prior sparse, window size list mismatch sparse scales!"
        # local-window run of every sparse scale (sparse_attn.py:915-938)
        self.local_inds: Dict[int, Tuple[torch.Tensor, int]] = {}
        for i in range(n_sparse):
            si = spsd_scale + 1 + i
            self.local_inds[si] = mb.local_group_runs(si, wind[i], self.bm, self.multiple_of, scales=self.scales)
        self.dense_colsum_attn = ops.dense_colsum_attn_s if speedup else ops.dense_colsum_attn_q
        self.indices = None
        self.counts = None
        self.out_cache = None

    def forward(self, q, k, v, scale, do_full_step: bool = False, inference_step: int = 0, scale_ind: int = 0, layer_ind: int = 0):
        if not GLOBAL_CONFIG["attn"]["is_enabled"]:
            return ops.dense_attn(q, k, v, scale)[0]
        top_keys = GLOBAL_CONFIG["attn"]["top_keys"]
        if do_full_step:                                           # sparse_attn.py:991-1051
            o, bs = self.dense_colsum_attn(q, k, v, scale)
            inds, counts = mb.topk_index_list(bs, top_keys, self.multiple_of, self.indices_pad_to)
            self.indices, self.counts = inds, counts
            if self.use_o_cache:
                # O_cache = O_dense + (-1) * delta(O) over the selected keys
                self.out_cache = ops.csp_attn(q, k, v, scale, inds, counts, o, -1)
            return o
        # sparse step, sparse_attn.py:1053-1144
        inds, counts = self.indices, self.counts
        s_count = int(counts[0, 0, 0])
        if inds.shape[0] != q.shape[0]:
            inds, counts = inds[:q.shape[0]], counts[:q.shape[0]]
        inds, counts = mb.map_inds_counts_across_scales(inds, s_count, cur_q_len=q.shape[-2], cur_k_len=k.shape[-2],
                                                        bm=self.bm, indices_pad_to=self.indices_pad_to)
        local_inds, local_count = self.local_inds[scale_ind]
        inds, counts = mb.append_local_run(inds, inds.shape[-1], local_inds, local_count,
                                           k_len=k.shape[-2], multiple_of=self.multiple_of)
        if scale_ind != len(self.scales) - 1:
            self.indices, self.counts = inds, counts               # cached for the next scale
        if self.use_o_cache:
            o = self.out_cache
            if o.shape[0] != q.shape[0]:
                o = o[:q.shape[0]]
            o = mb.upsample_ocache(o, o.shape[-2], q.shape[-2]).to(v.dtype)
        else:
            o = torch.zeros_like(q)
        return ops.csp_attn(q, k, v, scale, inds, counts, o, 1)

    __call__ = forward
