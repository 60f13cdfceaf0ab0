"""Device memory of the cache groups.

A paged group keeps, for each of its layers, keys as [pages, kv_heads, block_size, head_dim] (the
reference's layout, src/cuda/kv_cache.h:1-2) and values transposed inside the page, [pages,
kv_heads, head_dim, block_size]: eight consecutive tokens of one value dim are then 16 contiguous
bytes, which is exactly the operand a matrix instruction wants for P*V (the reduction runs over
tokens), just as eight dims of one token are for Q*K^T.  All layers of the group share one
allocation; a page id means the same page in every layer of the group.  A state group keeps one
slot per admitted request and layer.  Memory is zeroed once at construction and never on reuse:
a reused page holds its previous owner's data beyond the new owner's length, and only the
context length keeps it out of sight (src/cuda/kv_cache.cu:12-14).
"""
import torch

from ..parts.base import KVCacheNeed, StateNeed


class KVStorage:
    def __init__(self, group: int, need: KVCacheNeed, num_layers: int, num_blocks: int, block_size: int,
                 dtype: torch.dtype, device):
        self.group, self.need = group, need
        self.num_layers, self.num_blocks, self.block_size = num_layers, num_blocks, block_size
        self.value_dim = need.value_dim or need.head_dim
        per_layer = num_blocks * need.num_kv_heads * block_size * max(need.head_dim, self.value_dim)
        if num_blocks * block_size >= 2 ** 31 or per_layer > 2 ** 35:
            # slot numbers are 32-bit; the decode kernels keep offsets inside a layer's cache as 32 bits x 8 elements
            raise ValueError(f"cache group {group}: {num_blocks} pages of {block_size} tokens are more than the kernels "
                             f"address (at most 2^31 token slots and 2^35 elements of keys per layer)")
        if self.value_dim == need.head_dim:
            self.data = torch.zeros(num_layers, 2, num_blocks, need.num_kv_heads, block_size, need.head_dim,
                                    dtype=dtype, device=device)
            self._k, self._v = self.data[:, 0], self.data[:, 1]
        else:       # keys and values of different sizes: an allocation each
            self._k = torch.zeros(num_layers, num_blocks, need.num_kv_heads, block_size, need.head_dim, dtype=dtype, device=device)
            self._v = torch.zeros(num_layers, num_blocks, need.num_kv_heads, self.value_dim, block_size, dtype=dtype, device=device)
            self.data = self._k
        # pooled entries: 32-bit mean keys and values of blocks of ``pool`` tokens, kept with the page of a block's last token
        self.pool_entries = -(-block_size // need.pool) if need.pool > 0 else 0
        self._pk = self._pv = None
        if self.pool_entries:
            self._pk = torch.zeros(num_layers, num_blocks, need.num_kv_heads, self.pool_entries, need.head_dim,
                                   dtype=torch.float32, device=device)
            self._pv = torch.zeros(num_layers, num_blocks, need.num_kv_heads, self.pool_entries, self.value_dim,
                                   dtype=torch.float32, device=device)

    def k(self, layer: int) -> torch.Tensor:
        """[pages, kv_heads, block_size, head_dim]"""
        return self._k[layer]

    def v(self, layer: int) -> torch.Tensor:
        """[pages, kv_heads, value_dim, block_size]: read transposed"""
        n = self.need
        return self._v[layer].view(self.num_blocks, n.num_kv_heads, self.value_dim, self.block_size)

    def pooled_k(self, layer: int) -> torch.Tensor:
        """[pages, kv_heads, entries, head_dim], float32 (a need with pool > 0)"""
        return self._pk[layer]

    def pooled_v(self, layer: int) -> torch.Tensor:
        """[pages, kv_heads, entries, value_dim], float32"""
        return self._pv[layer]

    @property
    def bytes_per_block(self) -> int:
        return bytes_per_block(self.need, self.num_layers, self.block_size, self._k.dtype)

    @property
    def total_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self._k, self._v, self._pk, self._pv) if t is not None)

    def bytes_read(self, context: int) -> int:
        """Bytes a request with ``context`` tokens has a step read from this group: the keys and values of
        every layer, of the window's tokens where there is a window (and the pooled entries before it)."""
        n = self.need
        tokens = min(context, n.window) if n.window > 0 else context
        token_bytes = self.num_layers * n.num_kv_heads * (n.head_dim + self.value_dim) * self._k.element_size()
        pooled = 0
        if n.pool > 0 and n.window > 0 and context > n.window:
            pooled = ((context - n.window) // n.pool) * self.num_layers * n.num_kv_heads * (n.head_dim + self.value_dim) * 4
        return tokens * token_bytes + pooled


class StateStorage:
    def __init__(self, group: int, need: StateNeed, num_layers: int, num_slots: int, device):
        self.group, self.need = group, need
        self.num_layers, self.num_slots = num_layers, num_slots
        self.data = torch.zeros(num_layers, num_slots, *need.shape, dtype=need.dtype, device=device)

    def slots(self, layer: int) -> torch.Tensor:
        return self.data[layer]

    def bytes_read(self, context: int) -> int:
        """One slot of every layer, whatever the context."""
        return self.num_layers * (self.data[0, 0].numel() * self.data.element_size())

    @property
    def total_bytes(self) -> int:
        return self.data.numel() * self.data.element_size()


def bytes_per_block(need: KVCacheNeed, num_layers: int, block_size: int, dtype: torch.dtype) -> int:
    """layers * kv_heads * block_size * (head_dim + value_dim) * element size (src/cuda/kv_cache.h:20-23), and the
    page's pooled entries where the need has them."""
    vd = need.value_dim or need.head_dim
    tokens = num_layers * need.num_kv_heads * block_size * (need.head_dim + vd) * torch.empty((), dtype=dtype).element_size()
    entries = -(-block_size // need.pool) if need.pool > 0 else 0
    return tokens + num_layers * need.num_kv_heads * entries * (need.head_dim + vd) * 4
