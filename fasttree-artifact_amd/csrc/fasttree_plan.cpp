// Host planner of FastTree decode attention as a C-ABI library (libfasttree_plan.so): the cost
// model, the greedy tree splitter, the three-pass adaptation and the vnode metadata builder of
// kernel_bench/fasttree.py:30-262, producing element-for-element the lists the reference's Python
// produces.  No GPU code; built with the host compiler and -ffp-contract=off (the split decisions
// compare IEEE doubles evaluated left to right, as Python evaluates them).
//
// The declarations are in include/fasttree_plan.h.

#include "fasttree_plan.h"

#include <algorithm>
#include <cstdint>
#include <deque>
#include <new>
#include <vector>

namespace {

struct Params {
  double alpha, beta, gamma;
  int64_t tsq[2], tsk[2];
  int64_t g;
};

// Python's % for a positive modulus
inline int64_t floor_mod(int64_t a, int64_t m) {
  const int64_t r = a % m;
  return r < 0 ? r + m : r;
}

// kernel_bench/fasttree.py:30-35
inline int64_t pad_q(int64_t ts, int64_t n) { return ts - (floor_mod(n - 1, ts) + 1); }
inline int64_t pad_k(int64_t ts, int64_t n) { return std::max<int64_t>(0, ts - n); }

// kernel_bench/fasttree.py:38-45; products are formed left to right in double, as
// `alpha * CpadQ * g * nK` is in Python
inline double cost_mm(int64_t nq, int64_t nk, const Params& p) {
  const int phase = nq > p.tsq[1] ? 0 : 1;
  double q_waste = p.alpha * (double)pad_q(p.tsq[phase], nq);
  q_waste = q_waste * (double)p.g;
  q_waste = q_waste * (double)nk;
  double k_waste = p.beta * (double)pad_k(p.tsk[phase], nk);
  k_waste = k_waste * (double)nq;
  k_waste = k_waste * (double)p.g;
  return q_waste + k_waste;
}
// kernel_bench/fasttree.py:48-61
inline double cost_red(int64_t nql, const Params& p) { return p.gamma * (double)nql; }
inline double split_q_cost(int64_t cur, int64_t nql, int64_t lenv, int64_t lenl, const Params& p) {
  return cost_mm(cur - nql, lenv, p) + cost_mm(nql, lenl + lenv, p);
}
inline double split_k_cost(int64_t cur, int64_t nql, int64_t lenl, int64_t lenv, const Params& p) {
  const double shared = cost_mm(cur, lenv, p) + cost_mm(nql, lenl, p);
  return shared + cost_red(nql, p);
}

struct Tree {
  int n;
  const int32_t* parent;
  const int32_t* seqlen;
  const int32_t* num_children;
  const int64_t* req_offs;
  const int32_t* req_ids;
  int64_t nreq(int v) const { return req_offs[v + 1] - req_offs[v]; }
};

// kernel_bench/fasttree.py:64-96: breadth first from node 0, children in ascending id
std::vector<int32_t> tree_heuristic(const Tree& t, const std::vector<std::vector<int>>& children, const Params& p) {
  std::vector<int64_t> run_len(t.n);
  for (int v = 0; v < t.n; ++v) run_len[v] = t.seqlen[v];
  std::vector<int32_t> assignment(t.n, 0);
  std::deque<int> pending{0};
  while (!pending.empty()) {
    const int v = pending.front();
    pending.pop_front();
    int64_t attached = t.nreq(v);
    const int64_t lenv = run_len[v];
    for (int l : children[v]) {
      const int64_t nql = t.nreq(l), lenl = run_len[l];
      const double keep_shared = split_k_cost(attached, nql, lenl, lenv, p);
      const double go_private = split_q_cost(attached, nql, lenv, lenl, p);
      if (keep_shared > go_private) {
        assignment[l] = 1;
        attached -= nql;
        run_len[l] = lenl + lenv;
      }
      pending.push_back(l);
    }
  }
  return assignment;
}

// kernel_bench/fasttree.py:126-141.  The root's parent is -1, which indexes the last element in
// Python; the same element is touched here.
std::vector<std::vector<int32_t>> requests_per_node(const Tree& t, const std::vector<int32_t>& assignment) {
  std::vector<std::vector<int32_t>> served(t.n);
  std::deque<int> fifo;
  for (int v = 0; v < t.n; ++v)
    if (t.num_children[v] == 0) {
      fifo.push_back(v);
      served[v].assign(t.req_ids + t.req_offs[v], t.req_ids + t.req_offs[v + 1]);
    }
  std::vector<int64_t> waiting(t.n);
  for (int v = 0; v < t.n; ++v) waiting[v] = t.num_children[v];
  while (!fifo.empty()) {
    const int v = fifo.front();
    fifo.pop_front();
    const int up = t.parent[v] < 0 ? t.parent[v] + t.n : t.parent[v];
    if (assignment[v] == 0 && v != 0)
      served[up].insert(served[up].end(), t.req_ids + t.req_offs[v], t.req_ids + t.req_offs[v + 1]);
    waiting[up] -= 1;
    if (waiting[up] == 0) fifo.push_back(up);
  }
  return served;
}

// run length of the chain a node's vnodes attend (kernel_bench/fasttree.py:149-153)
int64_t chain_len(const Tree& t, const std::vector<int32_t>& assignment, int v) {
  int64_t total = t.seqlen[v];
  while (assignment[v] == 1) {
    v = t.parent[v];
    total += t.seqlen[v];
  }
  return total;
}

}  // namespace

struct ft_plan {
  std::vector<int32_t> arrays[FT_PLAN_ARRAYS];
};

extern "C" {

int ft_plan_create(int n_nodes, const int32_t* parent, const int32_t* seqlen, const int32_t* num_children,
                   const int64_t* req_offs, const int32_t* req_ids, const int64_t* kv_ptrs,
                   int batch_size, int num_kv_heads, const int32_t kv_split_sizes[2],
                   const int32_t para_threshs1[2], const int32_t para_threshs2[2],
                   double alpha, double beta, double gamma, const int32_t tsq[2], const int32_t tsk[2],
                   int kv_group_num, const int32_t* kv_slot_map, int64_t kv_slot_map_len, ft_plan** out) {
  if (!parent || !seqlen || !num_children || !req_offs || !kv_ptrs || !kv_split_sizes || !para_threshs1 ||
      !para_threshs2 || !tsq || !tsk || !out)
    return FT_PLAN_ERR_NULL_POINTER;
  if (n_nodes < 1 || batch_size < 0 || tsq[0] < 1 || tsq[1] < 1 || tsk[0] < 1 || tsk[1] < 1 ||
      kv_split_sizes[0] < 1 || kv_split_sizes[1] < 1)
    return FT_PLAN_ERR_ARGUMENT;
  for (int v = 0; v < n_nodes; ++v) {
    if (parent[v] >= n_nodes || (v > 0 && (parent[v] < 0 || parent[v] >= v)) || seqlen[v] < 0) return FT_PLAN_ERR_ARGUMENT;
    if (req_offs[v + 1] < req_offs[v]) return FT_PLAN_ERR_ARGUMENT;
  }
  if (req_offs[n_nodes] > 0 && !req_ids) return FT_PLAN_ERR_NULL_POINTER;
  for (int64_t i = 0; i < req_offs[n_nodes]; ++i)
    if (req_ids[i] < 0 || req_ids[i] >= batch_size) return FT_PLAN_ERR_ARGUMENT;

  try {
    const Tree t{n_nodes, parent, seqlen, num_children, req_offs, req_ids};
    std::vector<std::vector<int>> children(n_nodes);
    for (int v = 1; v < n_nodes; ++v) children[parent[v]].push_back(v);

    Params p{alpha, beta, gamma, {tsq[0], tsq[1]}, {tsk[0], tsk[1]}, kv_group_num};
    int64_t q_tiles[2] = {tsq[0], tsq[1]};
    int64_t kv_splits[2] = {kv_split_sizes[0], kv_split_sizes[0]};
    bool mutated = false;
    std::vector<int32_t> history;
    std::vector<int32_t> assignment;
    std::vector<std::vector<int32_t>> served;

    // kernel_bench/fasttree.py:163-188
    for (int attempt = 0; attempt < 3; ++attempt) {
      assignment = tree_heuristic(t, children, p);
      served = requests_per_node(t, assignment);
      int64_t blocks[2] = {0, 0};
      for (int v = 0; v < n_nodes; ++v) {
        const int64_t n = (int64_t)served[v].size();
        if (n == 0) continue;
        const int64_t kv_len = chain_len(t, assignment, v);
        const int phase = n > q_tiles[1] ? 0 : 1;
        // Python floor division; kv_len - 1 is -1 for an empty run
        const int64_t a = kv_len - 1, s = kv_splits[phase];
        const int64_t kv_parts = (a >= 0 ? a / s : -((-a + s - 1) / s)) + 1;
        blocks[phase] += kv_parts * ((n - 1) / q_tiles[phase] + 1);
      }
      const int64_t para[2] = {blocks[0] * num_kv_heads, blocks[1] * num_kv_heads};
      for (int ph = 0; ph < 2; ++ph) {
        if (para[ph] > INT32_MAX) return FT_PLAN_ERR_ARGUMENT;
        history.push_back((int32_t)para[ph]);
      }
      if (attempt == 0) {
        bool starved = false;
        for (int ph = 0; ph < 2; ++ph)
          if (0 < para[ph] && para[ph] < para_threshs1[ph]) {
            kv_splits[ph] = kv_split_sizes[1];
            starved = true;
          }
        if (!starved) break;
      } else if (attempt == 1) {
        int keep;
        if (0 < para[0] && para[0] < para_threshs2[0]) keep = 1;
        else if (0 < para[1] && para[1] < para_threshs2[1]) keep = 0;
        else break;
        q_tiles[0] = q_tiles[1] = q_tiles[keep];
        p.tsq[0] = p.tsq[1] = q_tiles[0];
        p.tsk[0] = p.tsk[1] = p.tsk[keep];
        mutated = true;
      }
    }

    // kernel_bench/fasttree.py:193-231: vnodes, nodes ascending, phase-0 query tile for every node
    std::vector<int32_t> kv_entries, kv_offs, kv_lens, q_entries, q_offs, q_lens;
    std::vector<int> chain;
    const int64_t q_tile = q_tiles[0];
    for (int v = 0; v < n_nodes; ++v) {
      const std::vector<int32_t>& reqs = served[v];
      const int64_t n = (int64_t)reqs.size();
      if (n == 0) continue;
      const int64_t kv_split = kv_splits[n > q_tiles[1] ? 0 : 1];
      chain.clear();
      int walk = v;
      chain.push_back(walk);
      while (assignment[walk] == 1) {
        walk = parent[walk];
        chain.push_back(walk);
      }
      const int64_t run_base = (int64_t)kv_entries.size();
      for (auto it = chain.rbegin(); it != chain.rend(); ++it)
        for (int64_t pos = kv_ptrs[*it]; pos < kv_ptrs[*it + 1]; ++pos) {
          if (pos < 0 || pos > INT32_MAX) return FT_PLAN_ERR_ARGUMENT;
          kv_entries.push_back((int32_t)pos);
        }
      const int64_t kv_len = (int64_t)kv_entries.size() - run_base;
      if ((int64_t)kv_entries.size() > INT32_MAX - FT_PLAN_ENTRY_PADDING) return FT_PLAN_ERR_ARGUMENT;
      for (int64_t kv_lo = 0; kv_lo < kv_len; kv_lo += kv_split) {
        const int64_t row_base = (int64_t)q_entries.size();
        if (row_base + n > INT32_MAX - FT_PLAN_ENTRY_PADDING) return FT_PLAN_ERR_ARGUMENT;
        q_entries.insert(q_entries.end(), reqs.begin(), reqs.end());
        const int64_t span = std::min(kv_lo + kv_split, kv_len) - kv_lo;
        for (int64_t q_lo = 0; q_lo < n; q_lo += q_tile) {
          kv_offs.push_back((int32_t)(run_base + kv_lo));
          kv_lens.push_back((int32_t)span);
          q_offs.push_back((int32_t)(row_base + q_lo));
          q_lens.push_back((int32_t)(std::min(q_lo + q_tile, n) - q_lo));
        }
      }
    }

    // kernel_bench/fasttree.py:233-244: scratch rows of every request, ascending
    std::vector<int32_t> req_lens(batch_size, 0), req_offs_out(batch_size, 0);
    for (int32_t r : q_entries) req_lens[r] += 1;
    int64_t acc = 0;
    for (int r = 0; r < batch_size; ++r) {
      req_offs_out[r] = (int32_t)acc;
      acc += req_lens[r];
    }
    std::vector<int32_t> req_entries((size_t)acc + FT_PLAN_ENTRY_PADDING, -1), cursor(req_offs_out);
    for (size_t row = 0; row < q_entries.size(); ++row) req_entries[cursor[q_entries[row]]++] = (int32_t)row;

    // kernel_bench/fasttree.py:246-259: stable partition, wide vnodes first
    const int64_t small = q_tiles[1];
    std::vector<int> order;
    order.reserve(q_lens.size());
    for (size_t i = 0; i < q_lens.size(); ++i)
      if (q_lens[i] > small) order.push_back((int)i);
    const int32_t n_wide = (int32_t)order.size();
    for (size_t i = 0; i < q_lens.size(); ++i)
      if (q_lens[i] <= small) order.push_back((int)i);
    auto permuted = [&](const std::vector<int32_t>& src) {
      std::vector<int32_t> dst(src.size());
      for (size_t i = 0; i < order.size(); ++i) dst[i] = src[order[i]];
      return dst;
    };

    if (kv_slot_map) {
      for (int32_t& e : kv_entries) {
        if (e >= kv_slot_map_len) return FT_PLAN_ERR_ARGUMENT;
        e = kv_slot_map[e];
      }
    }
    kv_entries.insert(kv_entries.end(), FT_PLAN_ENTRY_PADDING, -1);

    ft_plan* plan = new ft_plan;
    plan->arrays[FT_PLAN_KV_ENTRIES] = std::move(kv_entries);
    plan->arrays[FT_PLAN_KV_OFFS] = permuted(kv_offs);
    plan->arrays[FT_PLAN_KV_LENS] = permuted(kv_lens);
    plan->arrays[FT_PLAN_Q_ENTRIES] = std::move(q_entries);
    plan->arrays[FT_PLAN_Q_OFFS] = permuted(q_offs);
    plan->arrays[FT_PLAN_Q_LENS] = permuted(q_lens);
    plan->arrays[FT_PLAN_REQ_ENTRIES] = std::move(req_entries);
    plan->arrays[FT_PLAN_REQ_OFFS] = std::move(req_offs_out);
    plan->arrays[FT_PLAN_REQ_LENS] = std::move(req_lens);
    plan->arrays[FT_PLAN_NODE_ASSIGNMENTS] = std::move(assignment);
    plan->arrays[FT_PLAN_PARALLELISMS] = std::move(history);
    plan->arrays[FT_PLAN_PHASE_NODE_NUMS] = {n_wide, (int32_t)order.size() - n_wide};
    plan->arrays[FT_PLAN_PHASE_NODE_OFFSETS] = {0, n_wide};
    plan->arrays[FT_PLAN_Q_TILE_SIZES] = {(int32_t)q_tiles[0], (int32_t)q_tiles[1]};
    plan->arrays[FT_PLAN_KV_SPLIT_SIZES] = {(int32_t)kv_splits[0], (int32_t)kv_splits[1]};
    plan->arrays[FT_PLAN_KV_TILE_SIZES] = {(int32_t)p.tsk[0], (int32_t)p.tsk[1]};
    plan->arrays[FT_PLAN_TILES_REPLACED] = {mutated ? 1 : 0};
    *out = plan;
    return FT_PLAN_OK;
  } catch (const std::bad_alloc&) {
    return FT_PLAN_ERR_MEMORY;
  }
}

int64_t ft_plan_size(const ft_plan* plan, int which) {
  if (!plan || which < 0 || which >= FT_PLAN_ARRAYS) return -1;
  return (int64_t)plan->arrays[which].size();
}

int ft_plan_copy(const ft_plan* plan, int which, int32_t* dst, int64_t capacity) {
  if (!plan || which < 0 || which >= FT_PLAN_ARRAYS) return FT_PLAN_ERR_ARGUMENT;
  const std::vector<int32_t>& src = plan->arrays[which];
  if ((int64_t)src.size() > capacity) return FT_PLAN_ERR_ARGUMENT;
  if (!src.empty() && !dst) return FT_PLAN_ERR_NULL_POINTER;
  std::copy(src.begin(), src.end(), dst);
  return FT_PLAN_OK;
}

void ft_plan_destroy(ft_plan* plan) { delete plan; }

const char* ft_plan_version(void) { return "fasttree_plan 0.1"; }

}  // extern "C"
