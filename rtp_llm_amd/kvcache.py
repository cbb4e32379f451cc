"""Paged KV-cache layout helpers (host side, torch ops, device-agnostic).

The allocator contract is the reference's: a per-layer tensor
``[blocks, 2, nkv, page, hd]`` (bindings/OpDefs.h:24-28,201-202), K block = index 0,
V block = index 1 of dim 1 (pool index 2b / 2b+1, kv_cache_kernels.cu:58-61), plus an
fp32 scale plane ``[blocks, 2, nkv, page]`` for 8-bit caches (MHAKVCacheSpec.h:52-54).
Inside a block the layout is MI355-native (we own the writer and every reader):

    K block: [nkv][page][hd]     V block: [nkv][hd][page]

8-bit caches hold the codes offset-binary (code + 128, i.e. the int8 with its top bit flipped): the attention kernel widens
bytes by placing them under an fp16 exponent, which wants unsigned bytes.  write_tokens / read_tokens take and return the
signed codes.

The hot-path writer is the HIP kernel behind ``ops.rope_kv_write``; the functions here
are the slow-path equivalents used to import a prefilled cache (the prefill path itself
is out of scope this round) and by the tests to read the cache back.
"""
from typing import Optional, Tuple

import torch


def alloc_layer_cache(num_blocks: int, nkv: int, page: int, hd: int, int8: bool, device,
                      dtype: torch.dtype = torch.float16) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """dtype: element type of a 16-bit cache (fp16 or bf16 -- the activation dtype of the model); ignored for INT8."""
    dt = torch.int8 if int8 else dtype
    kv = torch.zeros(num_blocks, 2, nkv, page, hd, dtype=dt, device=device)
    sc = torch.ones(num_blocks, 2, nkv, page, dtype=torch.float32, device=device) if int8 else None
    return kv, sc


def _flip(x: torch.Tensor) -> torch.Tensor:
    """signed code <-> stored byte (top bit flipped)."""
    return torch.bitwise_xor(x, torch.tensor(-128, dtype=torch.int8, device=x.device))


def _views(kv_base: torch.Tensor):
    nb, _, nkv, page, hd = kv_base.shape
    flat = kv_base.view(nb, 2, nkv, page * hd)
    k = flat[:, 0].unflatten(-1, (page, hd))   # [nb, nkv, page, hd]
    v = flat[:, 1].unflatten(-1, (hd, page))   # [nb, nkv, hd, page]
    return k, v


def write_tokens(kv_base: torch.Tensor, scale_base: Optional[torch.Tensor], block_table_row: torch.Tensor, start: int,
                 K: torch.Tensor, V: torch.Tensor, k_scale: Optional[torch.Tensor] = None,
                 v_scale: Optional[torch.Tensor] = None) -> None:
    """Store tokens start..start+T-1 of one sequence.  K, V: [T, nkv, hd] in the cache dtype;
    k_scale, v_scale: [T, nkv] fp32 for an int8 cache."""
    page = kv_base.shape[3]
    T = K.shape[0]
    pos = torch.arange(start, start + T, device=kv_base.device)
    blk = block_table_row.to(kv_base.device).long()[pos // page]
    off = pos % page
    kview, vview = _views(kv_base)
    K, V = K.to(kv_base.device), V.to(kv_base.device)
    if kv_base.dtype == torch.int8:
        K, V = _flip(K), _flip(V)
    kview[blk, :, off, :] = K
    vview[blk, :, :, off] = V
    if scale_base is not None:
        scale_base[blk, 0, :, off] = k_scale.to(kv_base.device)
        scale_base[blk, 1, :, off] = v_scale.to(kv_base.device)


def read_tokens(kv_base: torch.Tensor, scale_base: Optional[torch.Tensor], block_table_row: torch.Tensor, ctx: int):
    """Natural view of the first ctx tokens of one sequence: (K, V [ctx,nkv,hd], k_scale, v_scale [ctx,nkv] or None)."""
    page = kv_base.shape[3]
    pos = torch.arange(ctx, device=kv_base.device)
    blk = block_table_row.to(kv_base.device).long()[pos // page]
    off = pos % page
    kview, vview = _views(kv_base)
    K, V = kview[blk, :, off, :], vview[blk, :, :, off]
    if scale_base is None:
        return K, V, None, None
    return _flip(K), _flip(V), scale_base[blk, 0, :, off], scale_base[blk, 1, :, off]


# --------------------------------------------------------------------------- pool management for the serving engine
class PagePool:
    """Free list of KV pages shared by all layers (page i of every layer belongs to the same owner).  A fresh pool hands out pages
    0, 1, 2, ...; a page that came back is the next one handed out."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError(f"PagePool: {num_pages} pages")
        self.num_pages = num_pages
        self._free = list(range(num_pages - 1, -1, -1))

    @property
    def free(self) -> int:
        return len(self._free)

    def take(self, n: int):
        if n > len(self._free):
            raise MemoryError(f"PagePool: {n} pages wanted, {len(self._free)} free of {self.num_pages}")
        out = [self._free.pop() for _ in range(n)]
        return out

    def give(self, pages):
        for p in pages:
            if not 0 <= p < self.num_pages or p in self._free:
                raise ValueError(f"PagePool: page {p} is not out")
            self._free.append(p)


class SlotPool(PagePool):
    """Fixed-size slots of per-sequence state (the recurrent layers' fp32 states): one per live sequence."""


class SequenceCache:
    """What one live sequence holds: its pages (in position order), its state slot, the number of tokens already run and the last of them
    (-1 before the first: models whose embedding looks at the previous token continue from it)."""

    def __init__(self, slot: int):
        self.pages, self.slot, self.length, self.last_token = [], slot, 0, -1


class CacheManager:
    """Pages and state slots of the live sequences of one engine.  `page` tokens per page; a sequence gets pages as it grows and gives
    everything back on release.  reserve: pages promised to admitted sequences for tokens they have not run yet (generation)."""

    def __init__(self, num_pages: int, page: int, num_slots: int):
        self.page = page
        self.pages, self.slots = PagePool(num_pages), SlotPool(num_slots)
        self.live = {}
        self._promised = {}

    def pages_for(self, tokens: int) -> int:
        return (tokens + self.page - 1) // self.page

    def can_admit(self, total_tokens: int) -> bool:
        return self.slots.free > 0 and self.pages.free - sum(self._promised.values()) >= self.pages_for(total_tokens)

    def admit(self, sid, reserve_tokens: int = 0) -> SequenceCache:
        if sid in self.live:
            raise KeyError(f"sequence {sid!r} is already live")
        if self.slots.free == 0:
            raise MemoryError(f"no state slot free for {sid!r} ({self.slots.num_pages} live sequences at most)")
        sc = SequenceCache(self.slots.take(1)[0])
        self.live[sid] = sc
        self._promised[sid] = self.pages_for(reserve_tokens)
        return sc

    def grow(self, sid, new_tokens: int) -> SequenceCache:
        """Make room for `new_tokens` more tokens of a live sequence (its length moves when the step has run: advance())."""
        sc = self.live[sid]
        need = self.pages_for(sc.length + new_tokens) - len(sc.pages)
        if need > 0:
            sc.pages += self.pages.take(need)
            self._promised[sid] = max(0, self._promised[sid] - need)
        return sc

    def advance(self, sid, new_tokens: int, last_token: Optional[int] = None):
        sc = self.live[sid]
        sc.length += new_tokens
        if last_token is not None:
            sc.last_token = int(last_token)

    def release(self, sid):
        sc = self.live.pop(sid)
        self._promised.pop(sid, None)
        self.pages.give(sc.pages)
        self.slots.give([sc.slot])
