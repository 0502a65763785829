"""Python entry points of the decode path: thin argument marshalling over the C ABI.

``fasttree_decode`` keeps the reference's positional signature
(kernel_bench/fasttree.py:582-604; called positionally at kernel_bench/benchmark.py:115-124
and with ``sm_scale=`` / ``logit_cap=`` keywords by the SGLang plugin, plugin.py:28-50).
Work is enqueued on torch's current stream; nothing is synchronised or allocated.
"""

from __future__ import annotations

import torch

from . import _lib

_DTYPES = {torch.float16: _lib.FT_DTYPE_F16, torch.bfloat16: _lib.FT_DTYPE_BF16}


def _dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise _lib.FastTreeLibraryError(f"unsupported dtype {t.dtype}: fp16 and bf16 only") from None


def _stream_handle(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _narrow_table_ptr(phase_node_nums):
    """Device pointer of the narrow vnodes' records a launch-order plan carries, or None."""
    table = getattr(phase_node_nums, "narrow_table", None)
    return table.data_ptr() if table is not None else None


def _prog_records_ptr(phase_node_nums):
    """Device pointer of the records of the block programs a launch-order plan carries, or None."""
    table = getattr(phase_node_nums, "prog_records", None)
    return table.data_ptr() if table is not None and getattr(phase_node_nums, "prog_table", None) is not None else None


def _req_table_ptr(phase_node_nums):
    """Device pointer of the per-request records for the merge launch, or None."""
    table = getattr(phase_node_nums, "req_table", None)
    return table.data_ptr() if table is not None else None


def _need_gpu(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise _lib.FastTreeLibraryError("fasttree_decode needs device tensors; there is no CPU path")


def _need_i32(*tensors):
    for t in tensors:
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise _lib.FastTreeLibraryError("index tensors must be contiguous int32")


def _need_inner_contiguous(*tensors):
    for t in tensors:
        if t.stride(-1) != 1:
            raise _lib.FastTreeLibraryError("the last dimension of q, k, v, o and the scratch must be contiguous")


def fasttree_decode(
    q, k_buffer, v_buffer, o,
    vnode_to_kv_entries, vnode_to_kv_offs, vnode_to_kv_lens,
    vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens,
    req_to_vnode_entries, req_to_vnode_offs, req_to_vnode_lens,
    mid_o, mid_lse,
    phase_node_nums, phase_node_offsets, phase_q_tile_sizes, phase_kv_tile_sizes,
    sm_scale, logit_cap=-1,
):
    """Tree-structured decode attention; the result is written into ``o``.

    ``logit_cap`` is accepted and ignored, as in the reference (fasttree.py:603).
    """
    assert q.shape[-1] == k_buffer.shape[-1]          # fasttree.py:437-438
    _need_gpu(q, k_buffer, v_buffer, o, mid_o, mid_lse, vnode_to_kv_entries)
    _need_inner_contiguous(q, k_buffer, v_buffer, o, mid_o, mid_lse)
    _need_i32(vnode_to_kv_entries, vnode_to_kv_offs, vnode_to_kv_lens, vnode_to_q_entries, vnode_to_q_offs,
              vnode_to_q_lens, req_to_vnode_entries, req_to_vnode_offs, req_to_vnode_lens)
    if k_buffer.dtype != q.dtype or v_buffer.dtype != q.dtype or o.dtype != q.dtype:
        raise _lib.FastTreeLibraryError("q, k, v and o must share one dtype")
    if mid_o.dtype != torch.float32 or mid_lse.dtype != torch.float32:
        raise _lib.FastTreeLibraryError("mid_o and mid_lse must be float32")
    lib = _lib.load()
    programs = getattr(phase_node_nums, "prog_table", None)
    narrow_table = _narrow_table_ptr(phase_node_nums)
    if (programs is not None or narrow_table is not None) and q.shape[-1] >= 32:
        # the launch was arranged as block programs (launch_schedule.block_programs)
        rc = lib.ft_decode_programs(
            q.data_ptr(), k_buffer.data_ptr(), v_buffer.data_ptr(), o.data_ptr(),
            q.stride(0), q.stride(1), k_buffer.stride(0), k_buffer.stride(1),
            v_buffer.stride(0), v_buffer.stride(1), o.stride(0), o.stride(1),
            vnode_to_kv_entries.data_ptr(), vnode_to_kv_offs.data_ptr(), vnode_to_kv_lens.data_ptr(),
            vnode_to_q_entries.data_ptr(), vnode_to_q_offs.data_ptr(), vnode_to_q_lens.data_ptr(),
            req_to_vnode_entries.data_ptr(), req_to_vnode_offs.data_ptr(), req_to_vnode_lens.data_ptr(),
            mid_o.data_ptr(), mid_o.stride(0), mid_o.stride(1), mid_lse.data_ptr(), mid_lse.stride(0),
            _lib.int32_pair(phase_node_nums), _lib.int32_pair(phase_node_offsets),
            programs.data_ptr() if programs is not None else None,
            int(phase_node_nums.num_programs) if programs is not None else 0,
            int(phase_node_nums.narrow_in_programs) if programs is not None else 0, narrow_table,
            _prog_records_ptr(phase_node_nums), _req_table_ptr(phase_node_nums),
            q.shape[0], q.shape[1], k_buffer.shape[1], q.shape[-1],
            float(sm_scale), _dtype_code(q), _stream_handle(q),
        )
        _lib.check(rc, "ft_decode_programs")
        return
    rc = lib.ft_decode(
        q.data_ptr(), k_buffer.data_ptr(), v_buffer.data_ptr(), o.data_ptr(),
        q.stride(0), q.stride(1), k_buffer.stride(0), k_buffer.stride(1),
        v_buffer.stride(0), v_buffer.stride(1), o.stride(0), o.stride(1),
        vnode_to_kv_entries.data_ptr(), vnode_to_kv_offs.data_ptr(), vnode_to_kv_lens.data_ptr(),
        vnode_to_q_entries.data_ptr(), vnode_to_q_offs.data_ptr(), vnode_to_q_lens.data_ptr(),
        req_to_vnode_entries.data_ptr(), req_to_vnode_offs.data_ptr(), req_to_vnode_lens.data_ptr(),
        mid_o.data_ptr(), mid_o.stride(0), mid_o.stride(1), mid_lse.data_ptr(), mid_lse.stride(0),
        _lib.int32_pair(phase_node_nums), _lib.int32_pair(phase_node_offsets),
        _lib.int32_pair(phase_q_tile_sizes), _lib.int32_pair(phase_kv_tile_sizes),
        q.shape[0], q.shape[1], k_buffer.shape[1], q.shape[-1],
        float(sm_scale), _dtype_code(q), _stream_handle(q),
    )
    _lib.check(rc, "ft_decode")


def fasttree_decode_static(q, k_buffer, v_buffer, o, vnode_to_kv_entries, vnode_to_kv_offs, vnode_to_kv_lens,
                           vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens, req_to_vnode_entries,
                           req_to_vnode_offs, req_to_vnode_lens, phase_node_nums, phase_node_offsets, sm_scale):
    """The decode call for callers that cannot allocate device memory (``ft_decode_static``):
    the partial results go to an array inside the library instead of ``mid_o`` / ``mid_lse``
    tensors, and neither this wrapper nor the library allocates on the device.  Not in the
    reference, whose caller allocates both buffers (kernel_bench/fasttree.py:264-269).

    Takes the lists of ``fasttree_preparation(launch_order=True)`` (``phase_node_nums`` carries
    the program table when there are wide vnodes).  Raises ``FastTreeLibraryError`` when the scratch rows
    do not fit the library's array (``ft_static_scratch_bytes()``, 64 MiB per device as built).  Calls that overlap on one device race
    on that array."""
    assert q.shape[-1] == k_buffer.shape[-1]
    _need_gpu(q, k_buffer, v_buffer, o, vnode_to_kv_entries)
    _need_inner_contiguous(q, k_buffer, v_buffer, o)
    _need_i32(vnode_to_kv_entries, vnode_to_kv_offs, vnode_to_kv_lens, vnode_to_q_entries, vnode_to_q_offs,
              vnode_to_q_lens, req_to_vnode_entries, req_to_vnode_offs, req_to_vnode_lens)
    if k_buffer.dtype != q.dtype or v_buffer.dtype != q.dtype or o.dtype != q.dtype:
        raise _lib.FastTreeLibraryError("q, k, v and o must share one dtype")
    lib = _lib.load()
    programs = getattr(phase_node_nums, "prog_table", None)
    rc = lib.ft_decode_static(
        q.data_ptr(), k_buffer.data_ptr(), v_buffer.data_ptr(), o.data_ptr(),
        q.stride(0), q.stride(1), k_buffer.stride(0), k_buffer.stride(1),
        v_buffer.stride(0), v_buffer.stride(1), o.stride(0), o.stride(1),
        vnode_to_kv_entries.data_ptr(), vnode_to_kv_offs.data_ptr(), vnode_to_kv_lens.data_ptr(),
        vnode_to_q_entries.data_ptr(), vnode_to_q_offs.data_ptr(), vnode_to_q_lens.data_ptr(),
        req_to_vnode_entries.data_ptr(), req_to_vnode_offs.data_ptr(), req_to_vnode_lens.data_ptr(),
        int(vnode_to_q_entries.numel()),
        _lib.int32_pair(phase_node_nums), _lib.int32_pair(phase_node_offsets),
        programs.data_ptr() if programs is not None else None,
        int(getattr(phase_node_nums, "num_programs", 0)) if programs is not None else 0,
        int(getattr(phase_node_nums, "narrow_in_programs", 0)) if programs is not None else 0,
        _narrow_table_ptr(phase_node_nums), _prog_records_ptr(phase_node_nums), _req_table_ptr(phase_node_nums),
        q.shape[0], q.shape[1], k_buffer.shape[1], q.shape[-1],
        float(sm_scale), _dtype_code(q), _stream_handle(q),
    )
    _lib.check(rc, "ft_decode_static")


def fasttree_decode_stage1(q, k_buffer, v_buffer, vnode_to_kv_entries, vnode_to_kv_offs, vnode_to_kv_lens,
                           vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens, sm_scale, mid_o, mid_lse,
                           phase_node_nums, phase_node_offsets, phase_q_tile_sizes, phase_kv_tile_sizes):
    """Stage 1 alone (both phases): fills ``mid_o`` / ``mid_lse``
    (the role of _fasttree_decode_stage1, kernel_bench/fasttree.py:416-479)."""
    _need_gpu(q, k_buffer, v_buffer, mid_o, mid_lse)
    lib = _lib.load()
    programs = getattr(phase_node_nums, "prog_table", None)
    narrow_table = _narrow_table_ptr(phase_node_nums)
    if (programs is not None or narrow_table is not None) and q.shape[-1] >= 32:
        rc = lib.ft_stage1_programs(
            q.data_ptr(), k_buffer.data_ptr(), v_buffer.data_ptr(),
            q.stride(0), q.stride(1), k_buffer.stride(0), k_buffer.stride(1), v_buffer.stride(0), v_buffer.stride(1),
            vnode_to_kv_entries.data_ptr(), vnode_to_kv_offs.data_ptr(), vnode_to_kv_lens.data_ptr(),
            vnode_to_q_entries.data_ptr(), vnode_to_q_offs.data_ptr(), vnode_to_q_lens.data_ptr(),
            mid_o.data_ptr(), mid_o.stride(0), mid_o.stride(1), mid_lse.data_ptr(), mid_lse.stride(0),
            _lib.int32_pair(phase_node_nums), _lib.int32_pair(phase_node_offsets),
            programs.data_ptr() if programs is not None else None,
            int(phase_node_nums.num_programs) if programs is not None else 0,
            int(phase_node_nums.narrow_in_programs) if programs is not None else 0, narrow_table,
            _prog_records_ptr(phase_node_nums),
            q.shape[1], k_buffer.shape[1], q.shape[-1], float(sm_scale), _dtype_code(q), _stream_handle(q),
        )
        _lib.check(rc, "ft_stage1_programs")
        return
    rc = lib.ft_stage1_phases(
        q.data_ptr(), k_buffer.data_ptr(), v_buffer.data_ptr(),
        q.stride(0), q.stride(1), k_buffer.stride(0), k_buffer.stride(1), v_buffer.stride(0), v_buffer.stride(1),
        vnode_to_kv_entries.data_ptr(), vnode_to_kv_offs.data_ptr(), vnode_to_kv_lens.data_ptr(),
        vnode_to_q_entries.data_ptr(), vnode_to_q_offs.data_ptr(), vnode_to_q_lens.data_ptr(),
        mid_o.data_ptr(), mid_o.stride(0), mid_o.stride(1), mid_lse.data_ptr(), mid_lse.stride(0),
        _lib.int32_pair(phase_node_nums), _lib.int32_pair(phase_node_offsets),
        _lib.int32_pair(phase_q_tile_sizes), _lib.int32_pair(phase_kv_tile_sizes),
        q.shape[1], k_buffer.shape[1], q.shape[-1], float(sm_scale), _dtype_code(q), _stream_handle(q),
    )
    _lib.check(rc, "ft_stage1_phases")


def fasttree_decode_phase(q, k_buffer, v_buffer, vnode_to_kv_entries, vnode_to_kv_offs, vnode_to_kv_lens,
                          vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens, sm_scale, mid_o, mid_lse,
                          node_num, node_offset, q_tile, kv_tile):
    """One phase of stage 1 on its own: what one iteration of the reference's launch loop does
    (kernel_bench/fasttree.py:443-479)."""
    _need_gpu(q, k_buffer, v_buffer, mid_o, mid_lse)
    lib = _lib.load()
    hq, hkv = q.shape[1], k_buffer.shape[1]
    rc = lib.ft_stage1(
        q.data_ptr(), k_buffer.data_ptr(), v_buffer.data_ptr(),
        q.stride(0), q.stride(1), k_buffer.stride(0), k_buffer.stride(1), v_buffer.stride(0), v_buffer.stride(1),
        vnode_to_kv_entries.data_ptr(), vnode_to_kv_offs.data_ptr(), vnode_to_kv_lens.data_ptr(),
        vnode_to_q_entries.data_ptr(), vnode_to_q_offs.data_ptr(), vnode_to_q_lens.data_ptr(),
        int(node_offset), int(node_num), hkv, hq // hkv, q.shape[-1], int(q_tile), int(kv_tile), float(sm_scale),
        mid_o.data_ptr(), mid_o.stride(0), mid_o.stride(1), mid_lse.data_ptr(), mid_lse.stride(0),
        _dtype_code(q), _stream_handle(q),
    )
    _lib.check(rc, "ft_stage1")


def fasttree_decode_stage2(req_to_vnode_entries, req_to_vnode_offs, req_to_vnode_lens, mid_o, mid_lse, o):
    """Stage 2 alone (the role of _fasttree_decode_stage2, kernel_bench/fasttree.py:549-579)."""
    _need_gpu(mid_o, mid_lse, o)
    lib = _lib.load()
    rc = lib.ft_stage2(
        req_to_vnode_entries.data_ptr(), req_to_vnode_offs.data_ptr(), req_to_vnode_lens.data_ptr(),
        mid_o.data_ptr(), mid_o.stride(0), mid_o.stride(1), mid_lse.data_ptr(), mid_lse.stride(0),
        o.data_ptr(), o.stride(0), o.stride(1), o.shape[0], o.shape[1], o.shape[2],
        _dtype_code(o), _stream_handle(o),
    )
    _lib.check(rc, "ft_stage2")


def gathered_decode(q, k_cache, v_cache, cache_seqlens, o, sm_scale, kv_split=512, mid_o=None, mid_lse=None):
    """Decode attention without prefix sharing over a per-request gathered cache
    ``[B, max_seqlen, Hkv, D]`` -- the baseline the tree path is compared with (the layout
    of kernel_bench/flash_attn_wrap.py:36-70).  Scratch is allocated when not passed."""
    _need_gpu(q, k_cache, v_cache, cache_seqlens, o)
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise _lib.FastTreeLibraryError("k_cache and v_cache must be contiguous")
    batch, width, hkv, d = k_cache.shape
    nsplit = (width + kv_split - 1) // kv_split
    hq = q.shape[1]
    if mid_o is None:
        mid_o = torch.empty((batch * nsplit, hq, d), dtype=torch.float32, device=q.device)
        mid_lse = torch.empty((batch * nsplit, hq), dtype=torch.float32, device=q.device)
    lib = _lib.load()
    rc = lib.ft_gathered_decode(
        q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), cache_seqlens.data_ptr(), o.data_ptr(),
        q.stride(0), q.stride(1), o.stride(0), o.stride(1),
        batch, width, hq, hkv, d, int(kv_split), float(sm_scale),
        mid_o.data_ptr(), mid_lse.data_ptr(), _dtype_code(q), _stream_handle(q),
    )
    _lib.check(rc, "ft_gathered_decode")
    return mid_o, mid_lse


def store_kv_cache(cache_k, cache_v, out_cache_loc, k_buffer, v_buffer):
    """``k_buffer[out_cache_loc] = cache_k; v_buffer[out_cache_loc] = cache_v`` in one launch on
    the current stream: the two indexed assignments of SGLang v0.2.13's
    ``RadixAttention.store_kv_cache``, the step that precedes the decode in the hook
    (fasttree_sglang_plugin_v0_2_13/plugin.py:26).

    ``cache_k`` / ``cache_v`` are ``[tokens, Hkv, D]`` (or ``[tokens, Hkv * D]``), ``out_cache_loc``
    int32 or int64 pool slots.  A slot outside the pool is skipped, not wrapped.
    """
    import torch

    _need_gpu(cache_k, cache_v, out_cache_loc, k_buffer, v_buffer)
    hkv, d = k_buffer.shape[1], k_buffer.shape[2]
    if v_buffer.shape[1:] != k_buffer.shape[1:] or v_buffer.dtype != k_buffer.dtype:
        raise _lib.FastTreeLibraryError("k_buffer and v_buffer must have the same heads, head size and dtype")
    cache_k = cache_k.view(-1, hkv, d)
    cache_v = cache_v.view(-1, hkv, d)
    if cache_k.dtype != k_buffer.dtype or cache_v.dtype != k_buffer.dtype:
        raise _lib.FastTreeLibraryError("the new rows must have the pools' dtype")
    _need_inner_contiguous(cache_k, cache_v, k_buffer, v_buffer)
    n = cache_k.shape[0]
    if cache_v.shape[0] != n or out_cache_loc.numel() != n:
        raise _lib.FastTreeLibraryError("cache_k, cache_v and out_cache_loc must name the same number of tokens")
    if out_cache_loc.dtype not in (torch.int32, torch.int64) or not out_cache_loc.is_contiguous():
        raise _lib.FastTreeLibraryError("out_cache_loc must be a contiguous int32 or int64 tensor")
    lib = _lib.load()
    rc = lib.ft_store_kv(
        cache_k.data_ptr(), cache_v.data_ptr(), cache_k.stride(0), cache_k.stride(1), cache_v.stride(0), cache_v.stride(1),
        out_cache_loc.data_ptr(), int(out_cache_loc.dtype == torch.int64), n,
        k_buffer.data_ptr(), v_buffer.data_ptr(), k_buffer.stride(0), k_buffer.stride(1),
        v_buffer.stride(0), v_buffer.stride(1), min(k_buffer.shape[0], v_buffer.shape[0]), hkv, d,
        _dtype_code(k_buffer), _stream_handle(k_buffer),
    )
    _lib.check(rc, "ft_store_kv")
