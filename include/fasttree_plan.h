/*
 * C ABI of libfasttree_plan.so: the host planner of FastTree decode attention (no GPU code).
 *
 * ft_plan_create() is what a foreign-function binding of the reference's planner would bind: it
 * replaces the host part of fasttree_preparation (kernel_bench/fasttree.py:111-262: greedy split
 * decisions of :64-96 with the cost model of :30-61, the three-pass adaptation of :163-188, the
 * vnode lists of :193-231, the per-request row lists of :233-244 and the phase partition of
 * :246-262) and produces, element for element, the lists the reference builds.  Placing the lists
 * on a device and allocating the fp32 scratch (:265-296) stays with the caller.
 *
 * The tree is passed as arrays indexed by node id (node 0 is the root, parent[0] = -1, a parent's
 * id is smaller than its children's): parent, seqlen, num_children as in KVTreeNode
 * (kernel_bench/kv_tree_simple.py:4-10), the per-node request lists in CSR form (req_offs has
 * n_nodes + 1 entries), and kv_ptrs[n_nodes + 1], the prefix sums of seqlen
 * (kernel_bench/flash_attn_wrap.py:13-22).  kv_slot_map (may be NULL) maps the logical token
 * position kv_ptrs[node] + t to the pool slot that holds it.
 *
 * All results are int32 arrays owned by the plan object; query their length with
 * ft_plan_size() and copy them out with ft_plan_copy().  Functions return FT_PLAN_OK (0) or a
 * negative FT_PLAN_ERR_* code.
 */
#ifndef FASTTREE_PLAN_H_
#define FASTTREE_PLAN_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ft_plan ft_plan;

enum { FT_PLAN_OK = 0, FT_PLAN_ERR_NULL_POINTER = -1, FT_PLAN_ERR_ARGUMENT = -2, FT_PLAN_ERR_MEMORY = -3 };

/* -1 entries appended to the two entry arrays (kernel_bench/fasttree.py:261-262) */
enum { FT_PLAN_ENTRY_PADDING = 32 };

/* result arrays; the first nine are the index arrays of the decode call, in its argument order */
enum {
  FT_PLAN_KV_ENTRIES = 0,      /* vnode_to_kv_entries, padded */
  FT_PLAN_KV_OFFS,             /* vnode_to_kv_offs */
  FT_PLAN_KV_LENS,             /* vnode_to_kv_lens */
  FT_PLAN_Q_ENTRIES,           /* vnode_to_q_entries: one scratch row per (request, kv split) */
  FT_PLAN_Q_OFFS,              /* vnode_to_q_offs */
  FT_PLAN_Q_LENS,              /* vnode_to_q_lens */
  FT_PLAN_REQ_ENTRIES,         /* req_to_vnode_entries, padded */
  FT_PLAN_REQ_OFFS,            /* req_to_vnode_offs */
  FT_PLAN_REQ_LENS,            /* req_to_vnode_lens */
  FT_PLAN_NODE_ASSIGNMENTS,    /* per node: 1 = the node absorbed its parent's run */
  FT_PLAN_PARALLELISMS,        /* two numbers per adaptation pass, the values the reference prints */
  FT_PLAN_PHASE_NODE_NUMS,     /* [wide vnodes, narrow vnodes] */
  FT_PLAN_PHASE_NODE_OFFSETS,  /* [0, wide vnodes] */
  FT_PLAN_Q_TILE_SIZES,        /* final Q_TILE_SIZE_PER_PHASE */
  FT_PLAN_KV_SPLIT_SIZES,      /* final KV_SPLIT_SIZE_PER_PHASE */
  FT_PLAN_KV_TILE_SIZES,       /* final params.TSKs */
  FT_PLAN_TILES_REPLACED,      /* [1] if the second pass replaced params.TSQs / TSKs (fasttree.py:181-186) */
  FT_PLAN_ARRAYS
};

const char* ft_plan_version(void);

int ft_plan_create(int n_nodes, const int32_t* parent, const int32_t* seqlen, const int32_t* num_children,
                   const int64_t* req_offs, const int32_t* req_ids, const int64_t* kv_ptrs,
                   int batch_size, int num_kv_heads, const int32_t kv_split_sizes[2],
                   const int32_t para_threshs1[2], const int32_t para_threshs2[2],
                   double alpha, double beta, double gamma, const int32_t tsq[2], const int32_t tsk[2],
                   int kv_group_num, const int32_t* kv_slot_map, int64_t kv_slot_map_len, ft_plan** out);

/* number of int32 elements of result array `which`, or -1 */
int64_t ft_plan_size(const ft_plan* plan, int which);

/* copies result array `which` into dst (capacity in elements) */
int ft_plan_copy(const ft_plan* plan, int which, int32_t* dst, int64_t capacity);

void ft_plan_destroy(ft_plan* plan);

#ifdef __cplusplus
}
#endif
#endif /* FASTTREE_PLAN_H_ */
