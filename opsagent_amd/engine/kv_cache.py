"""Paged KV cache manager with block-level prefix caching.

SURVEY.md §2b: "hipGraph-captured decode step, re-used across multi-turn
ReAct iterations — the loop at simple.go:394-615 re-sends full history each
turn; persistent KV across tool-call turns = the agent-turn-latency lever."

Mechanism: the cache is a pool of fixed-size token blocks
([num_blocks, block_size, Hk_local, D] bf16 per layer, sized against the
288 GB of HBM3E per MI355X). Each FULL block of a sequence is content-hashed
by its chain hash (hash of all token ids up to and including the block);
completed blocks are published to a hash table. A new request reuses the
longest prefix of published blocks — so when the ReAct loop re-sends the
growing conversation, only the new suffix is prefilled. Freed blocks stay
cached (refcount 0) in LRU order and are evicted on allocation pressure.
"""

from __future__ import annotations

import collections
from typing import Dict, List, Optional, Sequence, Tuple

import torch


class BlockAllocatorError(RuntimeError):
    pass


class PagedKVCache:
    def __init__(
        self,
        num_layers: int,
        num_kv_heads_local: int,
        head_dim: int,
        block_size: int,
        num_blocks: int,
        device: str,
        dtype: torch.dtype = torch.bfloat16,
        layer_shapes: Optional[Sequence[Optional[Tuple[int, int, int]]]] = None,
        prefix_caching: bool = True,
    ):
        """layer_shapes (optional) gives each layer's own (kv_heads, key dim,
        value dim), or None for a layer that keeps no keys and values (a
        recurrent mixer, or a layer that reads another layer's cache); a
        fourth element "prefix" says that the values ARE the first `value
        dim` channels of the keys (one key head): the value tensor is then a
        view of the key rows and takes no memory; a fourth element "vheads"
        with a fifth n says that there are n value heads (n divides kv_heads:
        key head g reads value head g mod n). Without layer_shapes every
        layer is [kv_heads, head_dim] for both. prefix_caching=False turns block publishing and reuse off: a
        model that also carries recurrent state cannot restart from cached
        keys alone."""
        assert block_size & (block_size - 1) == 0, "block_size must be a power of 2"
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.device = device
        self.prefix_caching = prefix_caching
        self.layers: List[Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]] = []
        if layer_shapes is None:
            layer_shapes = [(num_kv_heads_local, head_dim, head_dim)] * num_layers
        for shape in layer_shapes:
            if shape is None:
                self.layers.append((None, None))
                continue
            hk, kdim, vdim = shape[:3]
            k = torch.zeros(num_blocks, block_size, hk, kdim, dtype=dtype, device=device)
            if len(shape) > 3 and shape[3] == "prefix":
                assert hk == 1 and vdim <= kdim
                v = k[..., :vdim]
            elif len(shape) > 4 and shape[3] == "vheads":
                assert hk % shape[4] == 0
                v = torch.zeros(num_blocks, block_size, shape[4], vdim, dtype=dtype,
                                device=device)
            else:
                v = torch.zeros(num_blocks, block_size, hk, vdim, dtype=dtype, device=device)
            self.layers.append((k, v))
        # allocator state
        self._free: collections.deque[int] = collections.deque(range(num_blocks))
        self._ref: List[int] = [0] * num_blocks
        # prefix cache: chain_hash -> block_id; and reverse for eviction.
        # _block_tokens keeps each published block's OWN token slice so a
        # 64-bit chain-hash collision cannot silently alias wrong KV: the
        # chain hash binds the ancestry, the stored slice verifies the
        # block's content (O(block_size) per block, not O(prefix)).
        self._hash_to_block: Dict[int, int] = {}
        self._block_to_hash: List[Optional[int]] = [None] * num_blocks
        self._block_tokens: List[Optional[Tuple[int, ...]]] = [None] * num_blocks
        # LRU of refcount-0 cached blocks (evictable)
        self._evictable: "collections.OrderedDict[int, None]" = collections.OrderedDict()
        self.stats = {"reused_blocks": 0, "allocated_blocks": 0, "evictions": 0}

    # -- low-level allocator ----------------------------------------------
    def num_free(self) -> int:
        return len(self._free) + len(self._evictable)

    def _pop_free_block(self) -> int:
        if self._free:
            return self._free.popleft()
        if self._evictable:
            bid, _ = self._evictable.popitem(last=False)  # LRU
            h = self._block_to_hash[bid]
            if h is not None:
                del self._hash_to_block[h]
                self._block_to_hash[bid] = None
                self._block_tokens[bid] = None
            self.stats["evictions"] += 1
            return bid
        raise BlockAllocatorError("KV cache out of blocks")

    def alloc_block(self) -> int:
        bid = self._pop_free_block()
        self._ref[bid] = 1
        self.stats["allocated_blocks"] += 1
        return bid

    def retain(self, bid: int) -> None:
        if self._ref[bid] == 0:
            self._evictable.pop(bid, None)
        self._ref[bid] += 1

    def release(self, bid: int) -> None:
        assert self._ref[bid] > 0
        self._ref[bid] -= 1
        if self._ref[bid] == 0:
            if self._block_to_hash[bid] is not None:
                self._evictable[bid] = None  # keep content for prefix reuse
            else:
                self._free.append(bid)

    # -- prefix cache -------------------------------------------------------
    @staticmethod
    def chain_hash(prev: int, ids: Sequence[int]) -> int:
        return hash((prev, tuple(ids)))

    def lookup_prefix(self, token_ids: Sequence[int]) -> Tuple[List[int], int]:
        """Longest reusable prefix. Returns (block_ids retained, n_tokens).

        Never reuses the entire prompt: at least one token must be recomputed
        so the engine has a last-token hidden state to sample from.
        """
        bs = self.block_size
        blocks: List[int] = []
        h = 0
        if not self.prefix_caching:
            return blocks, 0
        max_full = (len(token_ids) - 1) // bs  # leave ≥1 token to prefill
        for i in range(max_full):
            h = self.chain_hash(h, token_ids[i * bs : (i + 1) * bs])
            bid = self._hash_to_block.get(h)
            if bid is None:
                break
            # collision guard: the hash indexes, token equality decides
            if self._block_tokens[bid] != tuple(token_ids[i * bs : (i + 1) * bs]):
                break
            blocks.append(bid)
        for bid in blocks:
            self.retain(bid)
        self.stats["reused_blocks"] += len(blocks)
        return blocks, len(blocks) * bs

    def publish_block(
        self, bid: int, chain_h: int, prefix_tokens: Tuple[int, ...]
    ) -> int:
        """Publish a full block under its chain hash. If an identical block
        (hash AND token-verified) is already cached, switch to it (dedup) and
        release ours. Returns the canonical block id."""
        existing = self._hash_to_block.get(chain_h)
        if existing is not None and existing != bid:
            if self._block_tokens[existing] == prefix_tokens:
                self.retain(existing)
                self.release(bid)
                return existing
            # hash collision with DIFFERENT content: evict the stale entry
            self._block_to_hash[existing] = None
            self._block_tokens[existing] = None
        self._hash_to_block[chain_h] = bid
        self._block_to_hash[bid] = chain_h
        self._block_tokens[bid] = prefix_tokens
        return bid


class StateSlotPool:
    """Fixed-size per-sequence state beside the paged keys and values: the
    recurrent matrix of a delta-rule mixer and the last inputs of causal
    short convolutions. One slot per live sequence; a slot is handed out at
    admission and returned when the sequence ends or is preempted.

    A slot is NOT cleared when it is reused: every kernel that reads state
    takes the sequence's start position and treats everything before
    position 0 as zero, so stale contents are never observed (and nothing
    has to be memset inside a captured graph).

    tensors[layer][name] is [num_slots, *shape] float32.
    """

    def __init__(self, num_slots: int, layer_shapes: Sequence[Dict[str, Tuple[int, ...]]],
                 device: str):
        self.num_slots = num_slots
        self.tensors: List[Dict[str, torch.Tensor]] = []
        for shapes in layer_shapes:
            self.tensors.append({
                name: torch.zeros(num_slots, *shape, dtype=torch.float32, device=device)
                for name, shape in shapes.items()
            })
        self._free: collections.deque[int] = collections.deque(range(num_slots))

    def num_free(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise BlockAllocatorError("out of state slots")
        return self._free.popleft()

    def release(self, slot: int) -> None:
        assert 0 <= slot < self.num_slots and slot not in self._free
        self._free.append(slot)


class SequenceState:
    """Per-sequence cache bookkeeping."""

    def __init__(self, cache: PagedKVCache, token_ids: List[int],
                 state_pool: Optional[StateSlotPool] = None):
        self.cache = cache
        self.state_pool = state_pool
        # recurrent/convolution state slot (None for pure-attention models)
        self.state_slot: Optional[int] = (
            state_pool.alloc() if state_pool is not None else None
        )
        self.token_ids = list(token_ids)  # prompt + generated
        self.blocks: List[int] = []
        self.num_cached = 0     # tokens whose KV is in cache
        self.chain_h = 0        # chain hash over published full blocks
        self.published = 0      # number of full blocks published

    def reuse_prefix(self) -> int:
        blocks, n = self.cache.lookup_prefix(self.token_ids)
        self.blocks = blocks
        self.num_cached = n
        self.published = len(blocks)
        h = 0
        bs = self.cache.block_size
        for i in range(len(blocks)):
            h = self.cache.chain_hash(h, self.token_ids[i * bs : (i + 1) * bs])
        self.chain_h = h
        return n

    def ensure_capacity(self, n_tokens: int) -> None:
        bs = self.cache.block_size
        need = (n_tokens + bs - 1) // bs
        while len(self.blocks) < need:
            self.blocks.append(self.cache.alloc_block())

    def slots_for(self, start: int, count: int) -> torch.Tensor:
        """Flat slot ids for token positions [start, start+count)."""
        bs = self.cache.block_size
        out = torch.empty(count, dtype=torch.int32)
        for i in range(count):
            pos = start + i
            out[i] = self.blocks[pos // bs] * bs + pos % bs
        return out

    def all_slots(self, upto: int) -> torch.Tensor:
        return self.slots_for(0, upto)

    def publish_full_blocks(self) -> None:
        """Publish newly-completed full blocks to the prefix cache."""
        if not self.cache.prefix_caching:
            return
        bs = self.cache.block_size
        full = self.num_cached // bs
        while self.published < full:
            i = self.published
            self.chain_h = self.cache.chain_hash(
                self.chain_h, self.token_ids[i * bs : (i + 1) * bs]
            )
            self.blocks[i] = self.cache.publish_block(
                self.blocks[i], self.chain_h,
                tuple(self.token_ids[i * bs : (i + 1) * bs]),
            )
            self.published += 1

    def free(self) -> None:
        for bid in self.blocks:
            self.cache.release(bid)
        self.blocks = []
        if self.state_slot is not None:
            self.state_pool.release(self.state_slot)
            self.state_slot = None
