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


class SparseDiffAttn(torch.nn.Module):
    """Constructor arguments as the reference's (models/sparvar/sparse_attn.py:866-873; constructed at
    basic_sparvar.py:255-259 as ``SparseDiffAttn(layer_num, layer_counter, use_o_cache=True, spsd_scale=...)``).
    ``layer_counter`` is any object with an ``increment()`` method (the reference's ``LayerCounter``) or None; it
    is advanced once per call, as the reference does (sparse_attn.py:1151,1163).  ``wind_size`` is accepted and
    unused: the reference overwrites it with ``GLOBAL_CONFIG['attn']['cs4a_ws']`` (sparse_attn.py:905-906)."""

    def __init__(self, layer_num: int = 0, layer_counter=None, use_o_cache: bool = True,
                 scales: Sequence[int] = mb.INFINITY_SCALES, spsd_scale: int = 10, wind_size: Optional[Sequence[int]] = None,
                 speedup: bool = False):
        super().__init__()
        if isinstance(layer_counter, bool):
            raise TypeError("the second argument is the layer counter (sparse_attn.py:867), not use_o_cache")
        self.layer_num = layer_num
        self.layer_counter = layer_counter
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
        self.count_host = 0
        self.out_cache = None

    def forward(self, q, k, v, scale, do_full_step: bool = False, inference_step: int = 0, scale_ind: int = 0, layer_ind: int = 0):
        out = self._fast_attention(q, k, v, scale, do_full_step, scale_ind)
        if self.layer_counter is not None:
            self.layer_counter.increment()
        return out

    def _fast_attention(self, q, k, v, scale, do_full_step: bool, scale_ind: int):
        if not GLOBAL_CONFIG["attn"]["is_enabled"]:
            return ops.dense_attn(q, k, v, scale)[0]
        top_keys = GLOBAL_CONFIG["attn"]["top_keys"]
        if do_full_step:                                           # sparse_attn.py:991-1051
            o, bs = self.dense_colsum_attn(q, k, v, scale)
            inds, counts = mb.topk_index_list(bs, top_keys, self.multiple_of, self.indices_pad_to, order="index", zero_tail=False)
            self.indices, self.counts = inds, counts
            self.count_host = mb.indices_count(top_keys, k.shape[-2], self.multiple_of)
            if self.use_o_cache:
                # O_cache = O_dense + (-1) * delta(O) over the selected keys
                self.out_cache = ops.csp_attn(q, k, v, scale, inds, counts, o, -1)
            return o
        # sparse step, sparse_attn.py:1053-1144
        inds, counts = self.indices, self.counts
        s_count = self.count_host                                  # the reference reads counts[0,0,0] back (a host sync)
        if inds.shape[0] != q.shape[0]:
            inds, counts = inds[:q.shape[0]], counts[:q.shape[0]]
        local_inds, local_count = self.local_inds[scale_ind]
        if local_inds.device != inds.device:
            local_inds = local_inds.to(inds.device)
            self.local_inds[scale_ind] = (local_inds, local_count)
        # group remap + clamp + local-run append + counts in one launch (sparse_attn.py:1056-1121)
        # (columns behind the list stay as allocated, as the reference's torch.empty padding, sparse_attn.py:1113-1117)
        inds, counts = ops.remap_concat_lists(inds, s_count, q.shape[-2], k.shape[-2], local_inds,
                                              bm=self.bm, indices_pad_to=self.indices_pad_to, zero_tail=False)
        assert int(inds.shape[-1]) >= s_count + local_count and (s_count + local_count) % self.multiple_of == 0, \
            f"after add local sparse index, mismatch multiple_of={self.multiple_of}"
        if scale_ind != len(self.scales) - 1:
            self.indices, self.counts = inds, counts               # cached for the next scale
            pad = self.indices_pad_to
            self.count_host = max(pad, (s_count + pad - 1) // pad * pad) + local_count
        if self.use_o_cache:
            o = self.out_cache
            if o.shape[0] != q.shape[0]:
                o = o[:q.shape[0]]
            # bilinear upsample of the cache fused into the attention epilogue (sparse_attn.py:1129-1142)
            return ops.csp_attn_upsampled(q, k, v, scale, inds, counts, o, 1)
        return ops.csp_attn(q, k, v, scale, inds, counts, torch.zeros_like(q), 1)

