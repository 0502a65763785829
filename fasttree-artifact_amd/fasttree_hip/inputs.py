"""Synthetic decode inputs for a KV tree: queries, the token-granular KV pool, the
logical-position -> pool-slot map, and (on request) the per-request gathered copy that
engines without prefix sharing read.

Mirrors the role of kernel_bench/flash_attn_wrap.py:5-79 (``qkv_preparation``) with
three additions the reference bench lacks: a seed, a shuffled pool (page size 1, every
token in a random slot) and a vectorised gather.  Values are drawn on the host from a
counter-based numpy generator so that the same seed gives the same bits everywhere.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import numpy as np
import torch

from .kv_tree import KVTreeNode, assign_requests, kv_prefix_sums, root_path


@dataclass
class DecodeInputs:
    Q: torch.Tensor                 # [B, Hq, D]
    K_pool: torch.Tensor            # [T, Hkv, D]  pool slot major
    V_pool: torch.Tensor            # [T, Hkv, D]
    KV_ptrs: List[int]              # n + 1 logical prefix sums
    slot_map: Optional[np.ndarray]  # int64 [T] logical position -> pool slot, None = identity
    path_tokens: List[np.ndarray]   # per request: pool slots of its root path, in order
    batch_size: int


def request_paths(tree_info: List[KVTreeNode], KV_ptrs, slot_map=None) -> List[np.ndarray]:
    """Pool slots each request attends, root first (the rows a gathered cache would hold,
    kernel_bench/flash_attn_wrap.py:43-67)."""
    out = []
    for index, node in enumerate(tree_info):
        if node.num_children != 0:
            continue
        idx = np.concatenate(
            [np.arange(KV_ptrs[n], KV_ptrs[n + 1], dtype=np.int64) for n in root_path(tree_info, index)]
        )
        out.append(idx if slot_map is None else slot_map[idx])
    return out


def _draw(rng: np.random.Generator, shape, dtype: torch.dtype, chunk_rows: int = 1 << 16) -> torch.Tensor:
    out = torch.empty(shape, dtype=dtype)
    flat = out.view(shape[0], -1) if len(shape) > 1 else out.view(-1, 1)
    for lo in range(0, shape[0], chunk_rows):
        hi = min(shape[0], lo + chunk_rows)
        block = rng.standard_normal((hi - lo, flat.shape[1]), dtype=np.float32)
        flat[lo:hi] = torch.from_numpy(block).to(dtype)
    return out


def make_decode_inputs(
    tree_info: List[KVTreeNode],
    num_qo_heads: int,
    num_kv_heads: int,
    head_dim: int,
    device="cuda",
    dtype: torch.dtype = torch.float16,
    seed: int = 0,
    shuffle_slots: bool = True,
    host_rng: bool = True,
) -> DecodeInputs:
    """Seeded N(0,1) Q/K/V for ``tree_info``; assigns request ids to the tree as a side
    effect (leaf order, as kernel_bench/flash_attn_wrap.py:24-33).

    Draw order: K (logical order), V (logical order), Q, then the slot permutation.
    With ``host_rng=False`` the values come from the device generator instead (fast for
    multi-GB pools, not bit-reproducible across machines).
    """
    batch = assign_requests(tree_info)
    ptrs = kv_prefix_sums(tree_info)
    total = ptrs[-1]
    if host_rng:
        rng = np.random.default_rng(seed)
        k_log = _draw(rng, (total, num_kv_heads, head_dim), dtype)
        v_log = _draw(rng, (total, num_kv_heads, head_dim), dtype)
        q = _draw(rng, (batch, num_qo_heads, head_dim), dtype)
        slot_map = rng.permutation(total).astype(np.int64) if shuffle_slots else None
        k_log, v_log, q = k_log.to(device), v_log.to(device), q.to(device)
    else:
        gen = torch.Generator(device=device)
        gen.manual_seed(seed)
        k_log = torch.randn((total, num_kv_heads, head_dim), device=device, dtype=dtype, generator=gen)
        v_log = torch.randn((total, num_kv_heads, head_dim), device=device, dtype=dtype, generator=gen)
        q = torch.randn((batch, num_qo_heads, head_dim), device=device, dtype=dtype, generator=gen)
        slot_map = np.random.default_rng(seed).permutation(total).astype(np.int64) if shuffle_slots else None

    if slot_map is None:
        k_pool, v_pool = k_log, v_log
    else:
        # pool[slot_map[p]] = logical[p]
        where = torch.from_numpy(slot_map).to(device)
        k_pool = torch.empty_like(k_log)
        v_pool = torch.empty_like(v_log)
        k_pool[where] = k_log
        v_pool[where] = v_log
        del k_log, v_log
    return DecodeInputs(
        Q=q, K_pool=k_pool, V_pool=v_pool, KV_ptrs=ptrs, slot_map=slot_map,
        path_tokens=request_paths(tree_info, ptrs, slot_map), batch_size=batch,
    )


def gather_per_request(inputs: DecodeInputs, max_seqlen: Optional[int] = None):
    """Per-request padded copy ``K_cache, V_cache [B, max_seqlen, Hkv, D]`` plus int32
    ``cache_seqlens [B]`` -- the layout engines without prefix sharing attend over
    (kernel_bench/flash_attn_wrap.py:36-70).  Padding rows are left uninitialised, as
    in the reference."""
    lens = [len(p) for p in inputs.path_tokens]
    width = max(lens) if max_seqlen is None else max_seqlen
    dev = inputs.K_pool.device
    shape = (inputs.batch_size, width) + tuple(inputs.K_pool.shape[1:])
    k_cache = torch.empty(shape, dtype=inputs.K_pool.dtype, device=dev)
    v_cache = torch.empty(shape, dtype=inputs.V_pool.dtype, device=dev)
    for r, slots in enumerate(inputs.path_tokens):
        where = torch.from_numpy(slots).to(dev)
        k_cache[r, : len(slots)] = inputs.K_pool[where]
        v_cache[r, : len(slots)] = inputs.V_pool[where]
    seqlens = torch.tensor(lens, dtype=torch.int32, device=dev)
    return k_cache, v_cache, seqlens


def qkv_preparation(tree_info, num_qo_heads, num_kv_heads, head_dim, device="cuda",
                    dtype=torch.float16, *, seed: int = 0):
    """Same positional signature and return tuple as kernel_bench/flash_attn_wrap.py:5-79:
    ``Q, K_cache, V_cache, cache_seqlens, K_tree_tensor, V_tree_tensor, KV_ptrs`` with a
    node-major (unshuffled) pool, as the reference bench builds it."""
    inp = make_decode_inputs(tree_info, num_qo_heads, num_kv_heads, head_dim, device, dtype,
                             seed=seed, shuffle_slots=False)
    k_cache, v_cache, seqlens = gather_per_request(inp)
    return inp.Q, k_cache, v_cache, seqlens, inp.K_pool, inp.V_pool, inp.KV_ptrs
