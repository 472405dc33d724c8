"""KV caches (reference cache.py): FP16 and Q4, contiguous [batch, max_seq_len, kv_heads, head_dim] per layer, or paged
views [pages, 256, kv_heads, head_dim] of the same storage (attn.py:504-505)."""
from __future__ import annotations

import torch

from .ext import none_tensor

PAGE_SIZE = 256                                           # generator/dynamic.py:33


class ExLlamaV2Cache:
    """FP16 cache (cache.py:230-300)."""

    def __init__(self, model, batch_size: int = 1, max_seq_len: int | None = None):
        cfg = model.config
        self.model = model
        self.batch_size = batch_size
        self.max_seq_len = max_seq_len or cfg.max_seq_len
        self.current_seq_len = 0
        shape = (batch_size, self.max_seq_len, cfg.num_key_value_heads, cfg.head_dim)
        n_layers = len(model.layers) if model.layers else cfg.num_hidden_layers          # layers held by this device
        self.key_states = [torch.zeros(shape, dtype=torch.float16, device=model.device) for _ in range(n_layers)]
        self.value_states = [torch.zeros(shape, dtype=torch.float16, device=model.device) for _ in range(n_layers)]

    def get_kv_state(self, layer_idx: int, batch_size: int, offset: int, width: int, page_size: int = 0,
                     cache_seqlens=None, block_table=None):
        return self.key_states[layer_idx], self.value_states[layer_idx]

    def store_kv_state(self, layer_idx: int, batch_size: int, offset: int, width: int, page_size: int = 0,
                       cache_seqlens=None, block_table=None):
        pass

    def paged_view(self, layer_idx: int):
        cfg = self.model.config
        k = self.key_states[layer_idx].view(-1, PAGE_SIZE, cfg.num_key_value_heads, cfg.head_dim)
        v = self.value_states[layer_idx].view(-1, PAGE_SIZE, cfg.num_key_value_heads, cfg.head_dim)
        return k, v

    def footprint(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.key_states + self.value_states)


class ExLlamaV2Cache_Q4(ExLlamaV2Cache):
    """Q4 cache (cache.py:409-606): uint8 codes + fp16 scales per 32 elements; one shared fp16 temp pair per device.
    get_kv_state dequantizes the live range into the temp, store_kv_state re-quantizes the touched blocks."""

    wbits = 4

    def __init__(self, model, batch_size: int = 1, max_seq_len: int | None = None):
        cfg = model.config
        self.model = model
        self.ext = model.ext
        self.batch_size = batch_size
        self.max_seq_len = max_seq_len or cfg.max_seq_len
        self.current_seq_len = 0
        kvh, hd, dev = cfg.num_key_value_heads, cfg.head_dim, model.device
        qshape = (batch_size, self.max_seq_len, kvh, hd // 2)
        sshape = (batch_size, self.max_seq_len, kvh, hd // 32)
        L = len(model.layers) if model.layers else cfg.num_hidden_layers
        self.key_states = [torch.zeros(qshape, dtype=torch.uint8, device=dev) for _ in range(L)]
        self.value_states = [torch.zeros(qshape, dtype=torch.uint8, device=dev) for _ in range(L)]
        self.key_scales = [torch.zeros(sshape, dtype=torch.float16, device=dev) for _ in range(L)]
        self.value_scales = [torch.zeros(sshape, dtype=torch.float16, device=dev) for _ in range(L)]
        tshape = (batch_size, self.max_seq_len, kvh, hd)
        self.temp_k = torch.zeros(tshape, dtype=torch.float16, device=dev)       # cache.py:464-469
        self.temp_v = torch.zeros(tshape, dtype=torch.float16, device=dev)

    def get_kv_state(self, layer_idx, batch_size, offset, width, page_size=0, cache_seqlens=None, block_table=None):
        """cache.py:472-514"""
        if width > 0 or page_size:
            self.ext.q_to_fp16_kv(self.key_states[layer_idx], self.temp_k, self.key_scales[layer_idx],
                                  self.value_states[layer_idx], self.temp_v, self.value_scales[layer_idx],
                                  batch_size, offset, width, page_size,
                                  cache_seqlens if cache_seqlens is not None else none_tensor,
                                  block_table if block_table is not None else none_tensor, self.wbits)
        return self.temp_k, self.temp_v

    def store_kv_state(self, layer_idx, batch_size, offset, width, page_size=0, cache_seqlens=None, block_table=None):
        """cache.py:517-556"""
        if width > 0:
            self.ext.fp16_to_q_kv(self.temp_k, self.key_states[layer_idx], self.key_scales[layer_idx],
                                  self.temp_v, self.value_states[layer_idx], self.value_scales[layer_idx],
                                  batch_size, offset, width, page_size,
                                  cache_seqlens if cache_seqlens is not None else none_tensor,
                                  block_table if block_table is not None else none_tensor, self.wbits)

    def paged_view(self, layer_idx):
        cfg = self.model.config
        return (self.temp_k.view(-1, PAGE_SIZE, cfg.num_key_value_heads, cfg.head_dim),
                self.temp_v.view(-1, PAGE_SIZE, cfg.num_key_value_heads, cfg.head_dim))

    def q4_views(self, layer_idx, paged: bool):
        """(k_codes, k_scales, v_codes, v_scales) of a layer for the fused Q4 attention kernel (attn_q4.hip): contiguous
        [b, T, KVH, .] or, paged, [pages, 256, KVH, .]."""
        ts = (self.key_states[layer_idx], self.key_scales[layer_idx], self.value_states[layer_idx], self.value_scales[layer_idx])
        if not paged:
            return ts
        kvh = self.model.config.num_key_value_heads
        return tuple(t.view(-1, PAGE_SIZE, kvh, t.shape[-1]) for t in ts)

    def footprint(self) -> int:
        ts = self.key_states + self.value_states + self.key_scales + self.value_scales
        return sum(t.numel() * t.element_size() for t in ts)


class PagePool:
    """Host-side allocator of cache pages and sequence slots for paged caches that several requests share.

    A sequence holds one slot (a row of the block table) and as many pages as its tokens need; both go back to the free lists when
    the sequence ends and are handed out again (most recently freed first).  The block table lives on the host and is mirrored to
    the device once per step (`device_table`), so kernels reach a token's row as
    `pages[block_table[slot, pos // page_size], pos % page_size]`."""

    def __init__(self, num_pages: int, page_size: int = PAGE_SIZE, max_seqs: int = 4, device="cuda:0"):
        if num_pages <= 0 or page_size <= 0 or max_seqs <= 0:
            raise ValueError("PagePool: sizes must be positive")
        self.num_pages, self.page_size, self.max_seqs = num_pages, page_size, max_seqs
        self.device = torch.device(device)
        self.free_pages = list(range(num_pages - 1, -1, -1))
        self.free_slots = list(range(max_seqs - 1, -1, -1))
        self.table = torch.zeros((max_seqs, num_pages), dtype=torch.int32)
        self.seq_pages = {}                                   # slot -> number of pages it holds
        self.seq_len = {}                                     # slot -> tokens cached
        self._dev_table = torch.zeros((max_seqs, num_pages), dtype=torch.int32, device=self.device)
        self._dirty = True

    def open(self) -> int:
        if not self.free_slots:
            raise RuntimeError(f"PagePool: all {self.max_seqs} sequence slots are in use")
        slot = self.free_slots.pop()
        self.seq_pages[slot] = 0
        self.seq_len[slot] = 0
        return slot

    def extend(self, slot: int, n_tokens: int) -> int:
        """Make room for n_tokens more tokens of the sequence; returns the position of the first of them."""
        start = self.seq_len[slot]
        need = -(-(start + n_tokens) // self.page_size)
        while self.seq_pages[slot] < need:
            if not self.free_pages:
                raise RuntimeError(f"PagePool: out of cache pages ({self.num_pages} x {self.page_size} tokens)")
            self.table[slot, self.seq_pages[slot]] = self.free_pages.pop()
            self.seq_pages[slot] += 1
            self._dirty = True
        self.seq_len[slot] = start + n_tokens
        return start

    def close(self, slot: int) -> None:
        for i in range(self.seq_pages.pop(slot) - 1, -1, -1):
            self.free_pages.append(int(self.table[slot, i]))
        del self.seq_len[slot]
        self.free_slots.append(slot)

    def device_table(self) -> torch.Tensor:
        if self._dirty:
            self._dev_table.copy_(self.table)
            self._dirty = False
        return self._dev_table


class LatentCache:
    """Paged cache of latent attention: one pool tensor [pages, page_size, kv_rank + rot_dim] per layer that OWNS its keys and
    values (a layer that attends over another layer's latents holds nothing: `owner[layer]` names whose rows it reads).  Rows are
    written by exl2_latent_append and read by exl2_latent_attn through the pool's block table."""

    def __init__(self, pool: PagePool, row_widths: dict, owner: dict, dtype):
        self.pool, self.owner, self.dtype = pool, dict(owner), dtype
        self.rows = {layer: torch.zeros((pool.num_pages, pool.page_size, width), dtype=dtype, device=pool.device)
                     for layer, width in row_widths.items()}

    def layer(self, layer_idx: int) -> torch.Tensor:
        return self.rows[self.owner[layer_idx]]

    def footprint(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.rows.values())


class PagedKV:
    """One attention layer's share of a PagePool: keys [pages, page, kv_heads, dim] and values [pages, page, kv_heads, vdim], and --
    for layers that see pooled blocks behind their window -- one mean key / mean value row per block of `block` tokens, kept with
    the page of the block's first token: [pages, ceil(page / block), kv_heads, dim | vdim]."""

    def __init__(self, pool: PagePool, kv_heads: int, dim: int, vdim: int, block: int, dtype):
        dev, P, n = pool.device, pool.page_size, pool.num_pages
        self.block = int(block)
        self.k = torch.zeros((n, P, kv_heads, dim), dtype=dtype, device=dev)
        self.v = torch.zeros((n, P, kv_heads, vdim), dtype=dtype, device=dev)
        self.k_pool = self.v_pool = None
        if self.block > 0:
            per_page = -(-P // self.block)
            self.k_pool = torch.zeros((n, per_page, kv_heads, dim), dtype=dtype, device=dev)
            self.v_pool = torch.zeros((n, per_page, kv_heads, vdim), dtype=dtype, device=dev)

    def tensors(self):
        return [t for t in (self.k, self.v, self.k_pool, self.v_pool) if t is not None]


class SlotState:
    """One recurrent layer's state per sequence slot of a PagePool: named tensors [max_seqs, ...], fp32 unless `dtype` says otherwise
    (int32 for remembered tokens).  Nothing is cleared when a slot is handed to a new sequence: the kernels start a sequence's first
    portion (position 0) from zeros by themselves."""

    def __init__(self, pool: PagePool, shapes: dict, dtype=torch.float32):
        self.t = {name: torch.zeros((pool.max_seqs,) + tuple(shape), dtype=dtype, device=pool.device)
                  for name, shape in shapes.items()}

    def __getitem__(self, name: str) -> torch.Tensor:
        return self.t[name]

    def tensors(self):
        return list(self.t.values())


class LayerStates:
    """What a stack of unlike mixers keeps between steps: per layer whatever its mixer's `make_state(pool, dtype)` built (PagedKV for
    attention, SlotState for recurrent mixers, None for a layer that reads another layer's rows), all over ONE PagePool, so a request's pages and its slot are handed out and taken
    back together."""

    def __init__(self, pool: PagePool, per_layer: dict, norm_states: dict | None = None):
        self.pool, self.per_layer = pool, dict(per_layer)
        # what the row-wise steps keep per slot: layer -> the norm in front of its mixer (token shift, input convolution),
        # (layer, "ff") -> the norm in front of its feed-forward, "embed" -> the embedding (previous token)
        self.norm_states = dict(norm_states or {})

    def layer(self, key):
        """key: a layer's index, or whatever a mixer that keeps several states names them by"""
        return self.per_layer[key]

    def norm_state(self, key):
        return self.norm_states.get(key)

    def footprint(self) -> int:
        states = list(self.per_layer.values()) + list(self.norm_states.values())
        return sum(t.numel() * t.element_size() for st in states if st is not None for t in st.tensors())
