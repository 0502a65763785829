/*
 * C ABI of libfasttree_hip.so: FastTree tree-structured decode attention for AMD
 * Instinct MI355X (gfx950).
 *
 * The functions below are what a foreign-function binding of the reference's decode
 * path would bind.  They take plain device pointers, element strides and sizes; they
 * allocate nothing, keep no pointer after returning, never synchronise the device and
 * enqueue all work on the HIP stream that is passed in.  Every function returns
 * FT_OK (0) or a negative FT_ERR_* code; ft_error_string() names a code.
 *
 * Conventions shared by all entry points
 *   - dtype: FT_DTYPE_F16 or FT_DTYPE_BF16, the element type of q, k, v and o.
 *   - q, o:  [batch, Hq, D]; k, v: [slots, Hkv, D]; the last dimension is contiguous,
 *     the two outer strides are given in elements and must be multiples of 8, and the
 *     base pointers must be 16-byte aligned.  K and V are separate allocations; their
 *     slot strides must lie in [0, 2^31).
 *   - mid_o [rows, Hq, D] and mid_lse [rows, Hq] are caller-owned fp32 scratch; stage 1
 *     overwrites them with the per-vnode partial result normalised by its own soft-max
 *     sum and with log-sum-exp of the scaled scores (natural log).  mid_o strides must
 *     be multiples of 4, the head stride of mid_lse is 1.
 *   - index arrays are contiguous int32 in device memory.  No element past the ranges
 *     named by the offset/length arrays is ever read.
 *   - D in {16, 32, 64, 128, 256} (the reference's set, kernel_bench/fasttree.py:439; 16 is computed as a
 *     zero-padded 32-dim contraction); Hq = Hkv * g with 1 <= g <= 64; sm_scale > 0.
 */
#ifndef FASTTREE_HIP_H_
#define FASTTREE_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* ft_stream_t; /* a hipStream_t; NULL = the null stream */

enum { FT_DTYPE_F16 = 0, FT_DTYPE_BF16 = 1 };

enum {
  FT_OK = 0,
  FT_ERR_NULL_POINTER = -1,
  FT_ERR_DTYPE = -2,
  FT_ERR_HEAD_DIM = -3,      /* reference: assert Lk in {16,32,64,128,256}, kernel_bench/fasttree.py:439 */
  FT_ERR_GROUP = -4,
  FT_ERR_ALIGNMENT = -5,
  FT_ERR_ARGUMENT = -6,
  FT_ERR_LAUNCH = -7,
  FT_ERR_SCRATCH = -8        /* ft_decode_static: more partial results than FT_STATIC_SCRATCH_BYTES hold */
};

/* Library version string, e.g. "fasttree_hip 0.1 (gfx950)". */
const char* ft_version(void);

/* Human-readable name of a return code. */
const char* ft_error_string(int code);

/*
 * Stage 1 for one phase: the partial attention of every vnode in
 * [vnode_begin, vnode_begin + vnode_count) against its KV slice, for all KV heads.
 * Replaces one launch of _fwd_fasttree_decode_stage1 by _fasttree_decode_stage1
 * (kernel_bench/fasttree.py:299-413, :443-479).  q_tile is the phase's query tile
 * (requests per vnode the planner used); vnodes with more requests are still computed
 * in full.  kv_tile is accepted for signature parity and does not change the result.
 */
int ft_stage1(const void* q, const void* k, const void* v,
              int64_t sq0, int64_t sq1, int64_t sk0, int64_t sk1, int64_t sv0, int64_t sv1,
              const int32_t* vnode_to_kv_entries, const int32_t* vnode_to_kv_offs,
              const int32_t* vnode_to_kv_lens, const int32_t* vnode_to_q_entries,
              const int32_t* vnode_to_q_offs, const int32_t* vnode_to_q_lens,
              int vnode_begin, int vnode_count, int num_kv_heads, int kv_group_num, int head_dim,
              int q_tile, int kv_tile, float sm_scale,
              float* mid_o, int64_t so0, int64_t so1, float* mid_lse, int64_t sl0,
              int dtype, ft_stream_t stream);

/*
 * Stage 1 for both phases in ONE launch: blocks for the wide phase first, then one wave per
 * (vnode, KV head) of the narrow phase, so the short narrow items fill the machine while the
 * wide blocks drain.  Replaces the whole of _fasttree_decode_stage1 (kernel_bench/fasttree.py:
 * 416-479); phase_* are its four 2-element python lists.
 */
int ft_stage1_phases(const void* q, const void* k, const void* v,
                     int64_t sq0, int64_t sq1, int64_t sk0, int64_t sk1, int64_t sv0, int64_t sv1,
                     const int32_t* vnode_to_kv_entries, const int32_t* vnode_to_kv_offs,
                     const int32_t* vnode_to_kv_lens, const int32_t* vnode_to_q_entries,
                     const int32_t* vnode_to_q_offs, const int32_t* vnode_to_q_lens,
                     float* mid_o, int64_t so0, int64_t so1, float* mid_lse, int64_t sl0,
                     const int32_t phase_node_nums[2], const int32_t phase_node_offsets[2],
                     const int32_t phase_q_tile_sizes[2], const int32_t phase_kv_tile_sizes[2],
                     int num_qo_heads, int num_kv_heads, int head_dim,
                     float sm_scale, int dtype, ft_stream_t stream);

/*
 * Stage 2: per (request, query head) log-sum-exp weighted merge of the request's
 * partial rows into o.  Replaces _fwd_fasttree_decoding_stage2 / _fasttree_decode_stage2
 * (kernel_bench/fasttree.py:482-579).
 */
int ft_stage2(const int32_t* req_to_vnode_entries, const int32_t* req_to_vnode_offs,
              const int32_t* req_to_vnode_lens,
              const float* mid_o, int64_t so0, int64_t so1, const float* mid_lse, int64_t sl0,
              void* o, int64_t oo0, int64_t oo1,
              int batch_size, int num_qo_heads, int head_dim, int dtype, ft_stream_t stream);

/*
 * The whole decode call: ft_stage1_phases, then ft_stage2.  Replaces
 * fasttree_decode (kernel_bench/fasttree.py:582-642); phase_* are its four 2-element
 * python lists.
 */
int ft_decode(const void* q, const void* k, const void* v, void* o,
              int64_t sq0, int64_t sq1, int64_t sk0, int64_t sk1, int64_t sv0, int64_t sv1,
              int64_t oo0, int64_t oo1,
              const int32_t* vnode_to_kv_entries, const int32_t* vnode_to_kv_offs,
              const int32_t* vnode_to_kv_lens, const int32_t* vnode_to_q_entries,
              const int32_t* vnode_to_q_offs, const int32_t* vnode_to_q_lens,
              const int32_t* req_to_vnode_entries, const int32_t* req_to_vnode_offs,
              const int32_t* req_to_vnode_lens,
              float* mid_o, int64_t so0, int64_t so1, float* mid_lse, int64_t sl0,
              const int32_t phase_node_nums[2], const int32_t phase_node_offsets[2],
              const int32_t phase_q_tile_sizes[2], const int32_t phase_kv_tile_sizes[2],
              int batch_size, int num_qo_heads, int num_kv_heads, int head_dim,
              float sm_scale, int dtype, ft_stream_t stream);

/*
 * Stage 1 of a launch that the host has arranged as block programs, and the whole decode call
 * with it (then ft_stage2).  No counterpart in the reference, which leaves the order and the
 * placement of its (vnode, KV head) blocks to the hardware dispatcher (kernel_bench/fasttree.py:
 * 443-479, grid = (node_num, head_num)).  One thread block per program and KV head walks the
 * program: prog_table holds four int32 per program in device memory -- first and end of its
 * vnodes within the range [phase_node_offsets[0], + phase_node_nums[0]) (served one after the
 * other, whole blocks), then first and count of its vnodes within the range
 * [phase_node_offsets[1], + phase_node_nums[1]) (served one wave each; a negative count means
 * before the others instead of after them).  The first narrow_in_programs vnodes of the second
 * range belong to programs; the rest of it is served one wave each by blocks of their own, as in
 * ft_stage1_phases, whatever their width.  The lists are otherwise those of ft_decode and
 * describe a complete plan without the table.  head_dim in {32, 64, 128, 256}.  The table is
 * trusted: it is not read on the host.
 *
 * narrow_table (or NULL) holds one record of 64 int32 per vnode of the second range, in the range's
 * order: the vnode's kv_off, kv_len, q_off and q_len as in the lists; then the requests of its first
 * 16 scratch rows (vnode_to_q_entries[q_off ...], unused entries anything); then the pool slots of its
 * first 32 tokens (vnode_to_kv_entries[kv_off + min(t, kv_len - 1)]); the rest is padding.  A wave that
 * serves such a vnode then starts with one memory round trip (the record) instead of two (the four
 * list entries, then the index and request lists) before it can ask for K/V rows.  The records must
 * agree with the lists; they are trusted like them.
 *
 * prog_records (or NULL) holds one record of 256 int32 per program: entries 0..3 the kv_off, kv_len,
 * q_off and q_len of the program's first vnode of the first range; entry 4 is 1 when the rest is filled
 * in (the program has such a vnode and it has at most 128 query rows = q_len * group), else 0; entries
 * 8..135 the requests of its scratch rows (vnode_to_q_entries[q_off ...]); entries 136..199 the pool slots
 * of its first 64 tokens (vnode_to_kv_entries[kv_off + min(t, kv_len - 1)]); the rest is padding.  A block
 * then asks for the query and K/V rows of its first vnode after one memory round trip (record and table
 * entry together) instead of three (table entry, list entries, request and slot lists).  Trusted like the
 * lists.
 *
 * req_table (or NULL; ft_decode_programs and ft_decode_static) holds one record of 16 int32 per
 * request for the second launch: req_to_vnode_lens[r], req_to_vnode_offs[r], then the first 14
 * entries of the request's part of req_to_vnode_entries (unused entries anything).  A block of the
 * second launch then knows which partial rows to ask for after one memory round trip instead of two
 * (length and offset, then the entries); entries beyond the fourteenth are read from the list.
 * Trusted like the lists.
 */
int ft_stage1_programs(const void* q, const void* k, const void* v,
                       int64_t sq0, int64_t sq1, int64_t sk0, int64_t sk1, int64_t sv0, int64_t sv1,
                       const int32_t* vnode_to_kv_entries, const int32_t* vnode_to_kv_offs,
                       const int32_t* vnode_to_kv_lens, const int32_t* vnode_to_q_entries,
                       const int32_t* vnode_to_q_offs, const int32_t* vnode_to_q_lens,
                       float* mid_o, int64_t so0, int64_t so1, float* mid_lse, int64_t sl0,
                       const int32_t phase_node_nums[2], const int32_t phase_node_offsets[2],
                       const int32_t* prog_table, int num_programs, int narrow_in_programs,
                       const int32_t* narrow_table, const int32_t* prog_records,
                       int num_qo_heads, int num_kv_heads, int head_dim,
                       float sm_scale, int dtype, ft_stream_t stream);

int ft_decode_programs(const void* q, const void* k, const void* v, void* o,
                       int64_t sq0, int64_t sq1, int64_t sk0, int64_t sk1, int64_t sv0, int64_t sv1,
                       int64_t oo0, int64_t oo1,
                       const int32_t* vnode_to_kv_entries, const int32_t* vnode_to_kv_offs,
                       const int32_t* vnode_to_kv_lens, const int32_t* vnode_to_q_entries,
                       const int32_t* vnode_to_q_offs, const int32_t* vnode_to_q_lens,
                       const int32_t* req_to_vnode_entries, const int32_t* req_to_vnode_offs,
                       const int32_t* req_to_vnode_lens,
                       float* mid_o, int64_t so0, int64_t so1, float* mid_lse, int64_t sl0,
                       const int32_t phase_node_nums[2], const int32_t phase_node_offsets[2],
                       const int32_t* prog_table, int num_programs, int narrow_in_programs,
                       const int32_t* narrow_table, const int32_t* prog_records, const int32_t* req_table,
                       int batch_size, int num_qo_heads, int num_kv_heads, int head_dim,
                       float sm_scale, int dtype, ft_stream_t stream);

/*
 * ft_decode_programs for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops and harnesses that forbid hipMalloc): the partial results live in a
 * device array of the library instead of mid_o / mid_lse buffers of the caller.  No counterpart
 * in the reference, whose caller allocates both (kernel_bench/fasttree.py:264-269).  The call
 * allocates and frees nothing on host-visible APIs: no hipMalloc, no hipFree, no library routine
 * that allocates.
 *
 * num_rows is the number of scratch rows the lists refer to (the length of vnode_to_q_entries);
 * it is trusted like the lists themselves: every vnode's q_off + q_len and every entry of
 * req_to_vnode_entries must lie below it, or the first launch writes outside the part of the
 * array that was checked against the capacity.
 * The array holds FT_STATIC_SCRATCH_BYTES (64 MiB unless the library was built with another
 * -DFT_STATIC_SCRATCH_BYTES=...) on every device of every process that loads the library, used or
 * not, for the life of the process; a call needs num_rows * num_qo_heads * head_dim * 4 bytes, rounded up to 256,
 * plus num_rows * num_qo_heads * 4, and returns FT_ERR_SCRATCH when that is more.  The first
 * call on a device looks up the array's address on that device (make it before a capture
 * starts); later calls on that device only launch the two kernels and take no lock.  All calls on one device
 * share the array: calls that overlap in time on one device (two streams, two threads) race on
 * it, and its contents are only meaningful between the two launches of one call.  Nothing in it
 * needs clearing: the first launch writes every row the second one reads.
 */
#ifndef FT_STATIC_SCRATCH_BYTES
#define FT_STATIC_SCRATCH_BYTES (64u << 20)
#endif
/* The capacity the loaded library was built with. */
int64_t ft_static_scratch_bytes(void);
int ft_decode_static(const void* q, const void* k, const void* v, void* o,
                     int64_t sq0, int64_t sq1, int64_t sk0, int64_t sk1, int64_t sv0, int64_t sv1,
                     int64_t oo0, int64_t oo1,
                     const int32_t* vnode_to_kv_entries, const int32_t* vnode_to_kv_offs,
                     const int32_t* vnode_to_kv_lens, const int32_t* vnode_to_q_entries,
                     const int32_t* vnode_to_q_offs, const int32_t* vnode_to_q_lens,
                     const int32_t* req_to_vnode_entries, const int32_t* req_to_vnode_offs,
                     const int32_t* req_to_vnode_lens, int64_t num_rows,
                     const int32_t phase_node_nums[2], const int32_t phase_node_offsets[2],
                     const int32_t* prog_table, int num_programs, int narrow_in_programs,
                     const int32_t* narrow_table, const int32_t* prog_records, const int32_t* req_table,
                     int batch_size, int num_qo_heads, int num_kv_heads, int head_dim,
                     float sm_scale, int dtype, ft_stream_t stream);

/*
 * Decode attention without prefix sharing over a per-request gathered, padded cache
 * k_cache, v_cache [batch, max_seqlen, Hkv, D] (contiguous) with cache_seqlens [batch]:
 * the layout the reference's comparison engines read (kernel_bench/flash_attn_wrap.py:36-70,
 * flashinfer_wrap.py:13-16).  Each request's sequence is cut into ceil(max_seqlen /
 * kv_split) pieces; mid_o / mid_lse need batch * ceil(max_seqlen / kv_split) rows.
 */
int ft_gathered_decode(const void* q, const void* k_cache, const void* v_cache,
                       const int32_t* cache_seqlens, void* o,
                       int64_t sq0, int64_t sq1, int64_t oo0, int64_t oo1,
                       int batch_size, int max_seqlen, int num_qo_heads, int num_kv_heads,
                       int head_dim, int kv_split, float sm_scale,
                       float* mid_o, float* mid_lse, int dtype, ft_stream_t stream);

/*
 * DeFT-Flatten, the tree-attention engine the reference's benchmark compares itself with
 * (kernel_bench/DeFT.py): ft_deft_stage1 replaces _fwd_DeFT_decode_stage1 / _DeFT_attn_stage_1
 * (DeFT.py:194-403), ft_deft_decode the whole of DeFT_decode (DeFT.py:489-560; its second stage,
 * DeFT.py:406-486, is the arithmetic of ft_stage2).  A vnode here is a subtree: a run of
 * consecutive tokens of the depth-first token order that may span several tree nodes
 * (vnode_to_kv_*), with the sorted set of requests that attend any of them (vnode_to_q_*).
 * causalmask holds, per subtree from causalmask_offset[subtree] on, kv_len 64-bit words for every
 * group of mask_len consecutive requests of the subtree's set: bit r of word t of group m says
 * that request m * mask_len + r of the set attends token t (DeFT.py:96-113).  One block per
 * (subtree, KV head); scores of tokens a request does not attend are set to a large negative value
 * before the soft-max; the normalised partial output is rounded to fp16 before it is stored to the
 * fp32 mid_o, as in the reference (DeFT.py:391).  mask_len is a power of two, at most 64, and at
 * least 128 / (3 * g) (the benchmark uses 64); head_dim in {32, 64, 128, 256}.
 */
int ft_deft_stage1(const void* q, const void* k, const void* v,
                   int64_t sq0, int64_t sq1, int64_t sk0, int64_t sk1, int64_t sv0, int64_t sv1,
                   const int32_t* vnode_to_kv_entries, const int32_t* vnode_to_kv_offs,
                   const int32_t* vnode_to_kv_lens, const int32_t* vnode_to_q_entries,
                   const int32_t* vnode_to_q_offs, const int32_t* vnode_to_q_lens,
                   const int64_t* causalmask, const int32_t* causalmask_offset,
                   int subtree_num, int num_qo_heads, int num_kv_heads, int head_dim, int mask_len, float sm_scale,
                   float* mid_o, int64_t so0, int64_t so1, float* mid_lse, int64_t sl0,
                   int dtype, ft_stream_t stream);

int ft_deft_decode(const void* q, const void* k, const void* v, void* o,
                   int64_t sq0, int64_t sq1, int64_t sk0, int64_t sk1, int64_t sv0, int64_t sv1,
                   int64_t oo0, int64_t oo1,
                   const int32_t* vnode_to_kv_entries, const int32_t* vnode_to_kv_offs,
                   const int32_t* vnode_to_kv_lens, const int32_t* vnode_to_q_entries,
                   const int32_t* vnode_to_q_offs, const int32_t* vnode_to_q_lens,
                   const int64_t* causalmask, const int32_t* causalmask_offset,
                   const int32_t* req_to_vnode_entries, const int32_t* req_to_vnode_offs,
                   const int32_t* req_to_vnode_lens,
                   float* mid_o, int64_t so0, int64_t so1, float* mid_lse, int64_t sl0,
                   int subtree_num, int batch_size, int num_qo_heads, int num_kv_heads, int head_dim,
                   int mask_len, float sm_scale, int dtype, ft_stream_t stream);

/*
 * The decode step's new K and V rows [num_tokens, Hkv, D] written to the pools at the slots
 * out_cache_loc[t] (int32, or int64 when loc_is_int64), both tensors in one launch on `stream`:
 * the two indexed assignments of SGLang v0.2.13's RadixAttention.store_kv_cache, which the hook
 * runs immediately before the decode (sglang_v0.2.13_bench/fasttree_sglang_plugin_v0_2_13/
 * plugin.py:26).  A token whose slot is outside [0, num_slots) is skipped.  Strides in elements,
 * multiples of 8; D a multiple of 8.  Work enqueued later on the same stream sees the rows.
 */
int ft_store_kv(const void* k_new, const void* v_new, int64_t kn0, int64_t kn1, int64_t vn0, int64_t vn1,
                const void* out_cache_loc, int loc_is_int64, int num_tokens,
                void* k_pool, void* v_pool, int64_t sk0, int64_t sk1, int64_t sv0, int64_t sv1,
                int64_t num_slots, int num_kv_heads, int head_dim, int dtype, ft_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* FASTTREE_HIP_H_ */
