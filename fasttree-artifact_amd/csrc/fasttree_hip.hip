// FastTree tree-structured decode attention for gfx950 (MI355X): the two device kernels
// and the C ABI declared in include/fasttree_hip.h.
//
// Stage 1 computes, for every virtual node (a set of <= Q_TILE requests that share one run
// of KV tokens) and every KV head, the soft-max partial of those requests' query heads
// over that run.  All query rows of a vnode (requests x GQA group) form the N side of
// 16x16x32 MFMA tiles; the gathered K rows are the M side of S^T = K Q^T and the gathered
// V rows are read back from LDS transposed (ds_read_b64_tr_b16) as the M side of
// O^T = V^T P^T, so the probabilities go from the first contraction's accumulators
// straight into the second contraction's B operand without leaving registers.
//
// Stage 2 merges each request's partials with their log-sum-exp weights using shuffles
// inside a group of D/4 lanes.
//
// Reference for the arithmetic: kernel_bench/fasttree.py:299-413 (stage 1), :482-546
// (stage 2), :582-642 (the call that chains them).

#include <hip/hip_runtime.h>
#include <algorithm>
#include <atomic>
#include <stdint.h>

#include "../../include/fasttree_hip.h"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWave * kWavesPerBlock;
constexpr int kTileTokens = 32;          // KV tokens per inner step (two 16-token MFMA row blocks)
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// ---------------------------------------------------------------------------------------
// Element-type traits: the 16-bit storage type only matters at the MFMA call and where
// fp32 probabilities / outputs are rounded to it.
// ---------------------------------------------------------------------------------------
struct F16 {
  static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ unsigned pack2(float lo, float hi) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(unsigned, v);
  }
  // acc + lo + hi of a packed pair, in fp32
  static __device__ __forceinline__ float add_pair(unsigned packed, float acc) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const h2 one = {(_Float16)1.f, (_Float16)1.f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, packed), one, acc, false);
  }
};
struct BF16 {
  static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ unsigned pack2(float lo, float hi) {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    b2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(unsigned, v);
  }
  static __device__ __forceinline__ float add_pair(unsigned packed, float acc) {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    const b2 one = {(__bf16)1.f, (__bf16)1.f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, packed), one, acc, false);
  }
};

// Wave-wide exchange helpers.  v_permlane{16,32}_swap exchanges the odd 16-lane rows
// (upper 32-lane half) of its first operand with the even rows (lower half) of its second;
// fed the same value twice it yields (value of the even row / lower half, value of the odd
// row / upper half) in every lane.  The two results are copied into scalars before they are
// reinterpreted: a bit cast applied directly to an element of the returned vector reads
// element 0 for both.
struct LanePair { float lo, hi; };
__device__ __forceinline__ LanePair halves16(float x) {
  const unsigned a = __builtin_bit_cast(unsigned, x);
  auto r = __builtin_amdgcn_permlane16_swap(a, a, false, false);
  const unsigned r0 = r[0], r1 = r[1];
  return {__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1)};
}
__device__ __forceinline__ LanePair halves32(float x) {
  const unsigned a = __builtin_bit_cast(unsigned, x);
  auto r = __builtin_amdgcn_permlane32_swap(a, a, false, false);
  const unsigned r0 = r[0], r1 = r[1];
  return {__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1)};
}
__device__ __forceinline__ float xor16_max(float x) { LanePair h = halves16(x); return fmaxf(h.lo, h.hi); }
__device__ __forceinline__ float xor32_max(float x) { LanePair h = halves32(x); return fmaxf(h.lo, h.hi); }
__device__ __forceinline__ float xor16_sum(float x) { LanePair h = halves16(x); return h.lo + h.hi; }
__device__ __forceinline__ float xor32_sum(float x) { LanePair h = halves32(x); return h.lo + h.hi; }
__device__ __forceinline__ float max3(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }
// Orders this wave's LDS traffic around a point where lanes read what other lanes of the
// same wave wrote.  LDS executes one wave's instructions in order, so no wait is needed;
// the fences only stop the compiler from moving accesses across.
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ float scale_from(float m_part, float m_all) {
  return (m_part == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_part - m_all);
}

struct Stage1Args {
  const char* q;
  const char* k;
  const char* v;
  int64_t sq0, sq1, sk0, sk1, sv0, sv1;  // element strides
  const int32_t* kv_entries;
  const int32_t* kv_offs;
  const int32_t* kv_lens;
  const int32_t* q_entries;
  const int32_t* q_offs;
  const int32_t* q_lens;
  int vnode_begin, vnode_count;    // vnodes served by wide blocks (or the whole range for the per-wave-staging kernel)
  int narrow_begin, narrow_count;  // vnodes of at most 16 rows
  int narrow_share;                // waves that share one narrow vnode: 1, 2 or 4
  int wide_rows;                   // query rows the planner's tile gives a wide vnode (host hint for wide_chunks)
  int wide_chunks;                 // blocks per (wide vnode, kv head); block c serves row pieces c, c + wide_chunks, ..
  int block_slots;                 // blocks of the fused kernel the device runs at a time
  // block programs written by the host (or null): four ints per program -- the wide vnodes
  // [first, end) of the wide range, then first and count of its narrow vnodes in the narrow range
  // (count < 0: they are served before the wide vnodes, else after them)
  const int32_t* prog_table;
  int num_programs;
  int narrow_in_programs;          // narrow vnodes (from narrow_begin) that programs serve
  // one record of kNarrowRecord ints per vnode of the narrow range, written by the host (or null):
  // what a wave needs to start on the vnode in one memory round trip instead of two -- the vnode's
  // four list entries, the requests of its rows and the pool slots of its first 32 tokens
  const int32_t* narrow_table;
  // one record of kProgRecord ints per program, written by the host (or null): what the block needs to
  // start on the program's first wide vnode -- see kProgRecord
  const int32_t* prog_records;
  int real_dim;                    // head dimension of the tensors; smaller than the kernel's D only for head_dim 16,
                                   // which the per-wave staging kernels compute as a zero-padded 32-dim contraction
  int g;
  int hkv;
  float scale_log2;  // sm_scale * log2(e)
  float* mid_o;
  int64_t so0, so1;
  float* mid_lse;
  int64_t sl0;
  // gathered (no-sharing) mode: vnode = (request, split) over a padded per-request cache
  const int32_t* cache_seqlens;
  int max_seqlen, kv_split, nsplit;
};

// How a kernel instance finds its vnode's slices.
struct VnodeView {
  int q_off;       // first scratch row
  int q_len;       // requests in this vnode
  int kv_len;      // tokens in the run
  int64_t kv_base; // tree mode: index into kv_entries; gathered mode: first cache row
};

template <bool GATHERED>
__device__ __forceinline__ VnodeView load_vnode(const Stage1Args& a, int vnode) {
  VnodeView w;
  if constexpr (GATHERED) {
    int req = vnode / a.nsplit, split = vnode - req * a.nsplit;
    int len = a.cache_seqlens[req] - split * a.kv_split;
    w.kv_len = len < 0 ? 0 : (len > a.kv_split ? a.kv_split : len);
    w.kv_base = (int64_t)req * a.max_seqlen + (int64_t)split * a.kv_split;
    w.q_off = vnode;
    w.q_len = 1;
  } else {
    w.q_off = a.q_offs[vnode];
    w.q_len = a.q_lens[vnode];
    w.kv_len = a.kv_lens[vnode];
    w.kv_base = a.kv_offs[vnode];
  }
  return w;
}

// Per-wave LDS staging of one 32-token tile.  Row pitches are chosen for the two read
// patterns: K rows are read 16 B per lane by 16 different rows at a time (pitch = 4 dwords
// mod 64 banks), V rows are read by ds_read_b64_tr_b16, where 16 lanes cover 4 rows x 32 B
// (pitch = 8 dwords mod 32 banks).
template <int D> struct TileGeom {
  static constexpr int kRowBytes = D * 2;
  static constexpr int kPitchK = kRowBytes + 16;
  static constexpr int kPitchV = kRowBytes + 32;
  static constexpr int kBytesK = kTileTokens * kPitchK;
  static constexpr int kBytesV = kTileTokens * kPitchV;
  static constexpr int kBytes = kBytesK + kBytesV;     // per wave
  static constexpr int kLanesPerRow = D / 8;           // 16-byte chunks in a row
  static constexpr int kRowsPerLoad = kWave / kLanesPerRow;
  static constexpr int kLoads = kTileTokens / kRowsPerLoad;
};

// Running soft-max state of one wave for NQB blocks of 16 query rows.  Accumulators are
// O^T tiles: lane l holds o[qb][db][j] = O[row 16*qb + l%16][dim 16*db + 4*(l/16) + j].
template <int D, int NQB> struct WaveState {
  f32x4 o[NQB][D / 16];
  float m[NQB];  // running max of scaled scores, log2 domain, identical in the 4 lanes of a row
  float l[NQB];  // running sum of this lane's own probabilities (reduced over lanes at the end)
};

// Query fragments of one wave (B operand of S^T = K Q^T): qf[qb][ks] holds, for row
// row0 + 16*qb + lane%16, the 8 dims 32*ks + 8*(lane/16) .. +7.  Rows past the vnode are zero.
template <int D, int NQB, bool GATHERED>
__device__ __forceinline__ void load_q_frags(const Stage1Args& a, const VnodeView& vn, int kvh, int row0,
                                             u32x4 (&qf)[NQB][D / 32]) {
  constexpr int KS = D / 32;
  const int lane = threadIdx.x & 63;
  const int p = lane & 15, c = lane >> 4;
  const int rows_total = vn.q_len * a.g;
#pragma unroll
  for (int qb = 0; qb < NQB; ++qb) {
    const int r = row0 + 16 * qb + p;
    const bool ok = r < rows_total;
    const int ri = ok ? r / a.g : 0;
    const int rj = ok ? r - ri * a.g : 0;
    const int64_t entry = ok ? (GATHERED ? (int64_t)(vn.q_off / a.nsplit) : (int64_t)a.q_entries[vn.q_off + ri]) : 0;
    const char* src = a.q + 2 * (entry * a.sq0 + (int64_t)(kvh * a.g + rj) * a.sq1 + 8 * c);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 z = {0u, 0u, 0u, 0u};
      qf[qb][ks] = ok && 32 * ks + 8 * c < a.real_dim ? *reinterpret_cast<const u32x4*>(src + 64 * ks) : z;
    }
  }
}

template <int D, int NQB>
__device__ __forceinline__ void reset_state(WaveState<D, NQB>& st) {
#pragma unroll
  for (int qb = 0; qb < NQB; ++qb) {
    st.m[qb] = -INFINITY;
    st.l[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < D / 16; ++db) st.o[qb][db] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
}

// every lane of a row gets the row's full probability sum
template <int D, int NQB>
__device__ __forceinline__ void finish_state(WaveState<D, NQB>& st) {
#pragma unroll
  for (int qb = 0; qb < NQB; ++qb) st.l[qb] = xor32_sum(xor16_sum(st.l[qb]));
}

// One 32-token step of a wave: scores of its NQB*16 rows against the tile staged at
// (ldsK, ldsV), online soft-max update, P.V.  `valid` (>= 1) is how many of the 32 tokens exist.
template <typename E, int D, int NQB>
__device__ __forceinline__ void tile_step(const char* ldsK, const char* ldsV, int valid, float sc,
                                          const u32x4 (&qf)[NQB][D / 32], WaveState<D, NQB>& st) {
  using G = TileGeom<D>;
  constexpr int KS = D / 32, DB = D / 16;
  const int lane = threadIdx.x & 63;
  const int p = lane & 15, c = lane >> 4;

  // ---- S^T = K Q^T : s[tb][qb][j] = score(token 16*tb + 4*c + j, row 16*qb + p)
  f32x4 s[2][NQB];
#pragma unroll
  for (int tb = 0; tb < 2; ++tb) {
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) s[tb][qb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const u32x4 kf = *reinterpret_cast<const u32x4*>(ldsK + (16 * tb + p) * G::kPitchK + 64 * ks + 16 * c);
#pragma unroll
      for (int qb = 0; qb < NQB; ++qb) s[tb][qb] = E::mfma(kf, qf[qb][ks], s[tb][qb]);
    }
  }

  // tokens past the end of the run score -inf (wave-uniform branch: only a run's last tile)
  if (valid < kTileTokens) {
#pragma unroll
    for (int tb = 0; tb < 2; ++tb)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (16 * tb + 4 * c + j >= valid) {
#pragma unroll
          for (int qb = 0; qb < NQB; ++qb) s[tb][qb][j] = -INFINITY;
        }
  }

  // Online soft-max with a lazily updated reference: a row's reference m only moves when the
  // row's running maximum exceeds it by more than kSlack (log2 units), so probabilities stay
  // below 2^kSlack -- exact in any case, since numerator and denominator share the reference --
  // and the accumulators are rescaled rarely instead of on almost every tile.
  constexpr float kSlack = 8.f;
  u32x4 pf[NQB];
#pragma unroll
  for (int qb = 0; qb < NQB; ++qb) {
    float mx = fmaxf(fmaxf(fmaxf(s[0][qb][0], s[0][qb][1]), fmaxf(s[0][qb][2], s[0][qb][3])),
                     fmaxf(fmaxf(s[1][qb][0], s[1][qb][1]), fmaxf(s[1][qb][2], s[1][qb][3])));
    mx = xor32_max(xor16_max(mx)) * sc;      // sc > 0; finite: the tile holds at least one token
    const float m_old = st.m[qb];
    const bool grow = mx > m_old + kSlack;   // also true on the first tile (m_old = -inf)
    if (__builtin_amdgcn_ballot_w64(grow)) {
      const float m_new = grow ? mx : m_old;
      const float alpha = __builtin_amdgcn_exp2f(m_old - m_new);
      st.l[qb] *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db) st.o[qb][db] *= alpha;
      st.m[qb] = m_new;
    }
    const float neg_m = -st.m[qb];
    float x[8];
    float sum = 0.f;
#pragma unroll
    for (int tb = 0; tb < 2; ++tb)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[4 * tb + j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[tb][qb][j], sc, neg_m));
        sum += x[4 * tb + j];
      }
    st.l[qb] += sum;
    pf[qb] = u32x4{E::pack2(x[0], x[1]), E::pack2(x[2], x[3]), E::pack2(x[4], x[5]), E::pack2(x[6], x[7])};
  }

  // ---- O^T += V^T P^T : A operand rows = dims 16*db + p, k slots = the 8 tokens this lane's P holds
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    const char* va = ldsV + (4 * c + (p >> 2)) * G::kPitchV + 2 * (16 * db + 4 * (p & 3));
    const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)(va));
    const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) i16x4*)(va + 16 * G::kPitchV));
    const u32x2 lo2 = __builtin_bit_cast(u32x2, lo), hi2 = __builtin_bit_cast(u32x2, hi);
    const u32x4 vf = {lo2[0], lo2[1], hi2[0], hi2[1]};
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) st.o[qb][db] = E::mfma(vf, pf[qb], st.o[qb][db]);
  }
}

// One wave attends NQB*16 query rows to tokens [tile0*32, ...) in steps of tile_step_n tiles,
// staging each tile in its own LDS area.  Rows travel global -> registers -> LDS; the next tile
// is in flight while a tile is consumed.  (Used for head_dim 256 only.)
template <typename E, int D, int NQB, bool GATHERED>
__device__ __forceinline__ void wave_attend(const Stage1Args& a, const VnodeView& vn, int kvh, int row0,
                                            int tile0, int tile_step_n, char* lds, WaveState<D, NQB>& st) {
  using G = TileGeom<D>;
  const int lane = threadIdx.x & 63;
  char* ldsK = lds;
  char* ldsV = lds + G::kBytesK;

  u32x4 qf[NQB][D / 32];
  load_q_frags<D, NQB, GATHERED>(a, vn, kvh, row0, qf);
  reset_state<D, NQB>(st);

  const int ntiles = (vn.kv_len + kTileTokens - 1) / kTileTokens;
  if (tile0 >= ntiles) return;

  // rows by 16-byte chunks, coalesced per row
  const int ld_row = lane / G::kLanesPerRow, ld_chunk = lane % G::kLanesPerRow;
  const char* kbase = a.k + 2 * ((int64_t)kvh * a.sk1) + 16 * ld_chunk;
  const char* vbase = a.v + 2 * ((int64_t)kvh * a.sv1) + 16 * ld_chunk;
  auto load_slots = [&](int tile, int (&slot)[G::kLoads]) {
#pragma unroll
    for (int i = 0; i < G::kLoads; ++i) {
      const int t = tile * kTileTokens + i * G::kRowsPerLoad + ld_row;
      slot[i] = -1;
      if (tile < ntiles && t < vn.kv_len) slot[i] = GATHERED ? t : a.kv_entries[vn.kv_base + t];
    }
  };
  auto load_rows = [&](const int (&slot)[G::kLoads], u32x4 (&kreg)[G::kLoads], u32x4 (&vreg)[G::kLoads]) {
#pragma unroll
    for (int i = 0; i < G::kLoads; ++i) {
      u32x4 z = {0u, 0u, 0u, 0u};
      kreg[i] = z;
      vreg[i] = z;
      if (slot[i] >= 0 && 8 * ld_chunk < a.real_dim) {   // (chunks past a 16-dim row stay zero)
        const int64_t srow = GATHERED ? (vn.kv_base + slot[i]) : (int64_t)slot[i];
        kreg[i] = *reinterpret_cast<const u32x4*>(kbase + 2 * srow * a.sk0);
        vreg[i] = *reinterpret_cast<const u32x4*>(vbase + 2 * srow * a.sv0);
      }
    }
  };
  auto stage = [&](const u32x4 (&kreg)[G::kLoads], const u32x4 (&vreg)[G::kLoads]) {
#pragma unroll
    for (int i = 0; i < G::kLoads; ++i) {
      const int row = i * G::kRowsPerLoad + ld_row;
      *reinterpret_cast<u32x4*>(ldsK + row * G::kPitchK + 16 * ld_chunk) = kreg[i];
      *reinterpret_cast<u32x4*>(ldsV + row * G::kPitchV + 16 * ld_chunk) = vreg[i];
    }
    wave_lds_fence();
  };

  int slot[G::kLoads];
  u32x4 kreg[G::kLoads], vreg[G::kLoads];
  load_slots(tile0, slot);
  load_rows(slot, kreg, vreg);
  for (int tile = tile0; tile < ntiles; tile += tile_step_n) {
    stage(kreg, vreg);
    if (tile + tile_step_n < ntiles) {
      load_slots(tile + tile_step_n, slot);
      load_rows(slot, kreg, vreg);
    }
    tile_step<E, D, NQB>(ldsK, ldsV, vn.kv_len - tile * kTileTokens, a.scale_log2, qf, st);
    wave_lds_fence();
  }
  finish_state<D, NQB>(st);
}

template <int D, int NQB>
__device__ __forceinline__ void write_partials(const Stage1Args& a, const VnodeView& vn, int kvh, int row0,
                                               const WaveState<D, NQB>& st) {
  constexpr int DB = D / 16;
  const int lane = threadIdx.x & 63;
  const int p = lane & 15, c = lane >> 4;
  const int rows_total = vn.q_len * a.g;
#pragma unroll
  for (int qb = 0; qb < NQB; ++qb) {
    const int r = row0 + 16 * qb + p;
    if (r >= rows_total) continue;
    const int ri = r / a.g, rj = r - ri * a.g;
    const int64_t row = vn.q_off + ri;
    const int head = kvh * a.g + rj;
    const float l = st.l[qb];
    const float inv = l > 0.f ? 1.f / l : 0.f;
    float* dst = a.mid_o + row * a.so0 + (int64_t)head * a.so1 + 4 * c;
#pragma unroll
    for (int db = 0; db < DB; ++db)
      if (16 * db < a.real_dim) *reinterpret_cast<f32x4*>(dst + 16 * db) = st.o[qb][db] * inv;
    if (c == 0) a.mid_lse[row * a.sl0 + head] = l > 0.f ? (__builtin_amdgcn_logf(l) + st.m[qb]) * kLn2 : -INFINITY;
  }
}

// Merge of the four waves' states of one block (each over the same rows, different tokens)
// into wave 0, pairwise through LDS: waves {2,3} -> {0,1}, then wave 1 -> wave 0.
template <int D, int NQB>
__device__ __forceinline__ void merge_waves(float* xchg, WaveState<D, NQB>& st) {
  constexpr int NV = NQB * (D / 16) * 4 + 2 * NQB;  // floats of state per lane
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
  for (int half = 2; half >= 1; half >>= 1) {
    __syncthreads();
    if (wave >= half && wave < 2 * half) {
      float* dst = xchg + (size_t)(wave - half) * NV * kWave + lane;
      int n = 0;
#pragma unroll
      for (int qb = 0; qb < NQB; ++qb) {
        dst[(n++) * kWave] = st.m[qb];
        dst[(n++) * kWave] = st.l[qb];
#pragma unroll
        for (int db = 0; db < D / 16; ++db)
#pragma unroll
          for (int j = 0; j < 4; ++j) dst[(n++) * kWave] = st.o[qb][db][j];
      }
    }
    __syncthreads();
    if (wave < half) {
      const float* src = xchg + (size_t)wave * NV * kWave + lane;
      int n = 0;
#pragma unroll
      for (int qb = 0; qb < NQB; ++qb) {
        const float m2 = src[(n++) * kWave];
        const float l2 = src[(n++) * kWave];
        const float m = fmaxf(st.m[qb], m2);
        const float a1 = scale_from(st.m[qb], m), a2 = scale_from(m2, m);
        st.l[qb] = st.l[qb] * a1 + l2 * a2;
        st.m[qb] = m;
#pragma unroll
        for (int db = 0; db < D / 16; ++db)
#pragma unroll
          for (int j = 0; j < 4; ++j) st.o[qb][db][j] = st.o[qb][db][j] * a1 + src[(n++) * kWave] * a2;
      }
    }
  }
}

// SPLIT_WAVES = true : one block per (vnode, kv head); its 4 waves take every 4th KV tile and
//                      their states are merged through LDS (wide vnodes, long runs).
// SPLIT_WAVES = false: one wave per (vnode, kv head), 4 vnodes per block (narrow vnodes).
template <typename E, int D, int NQB, bool SPLIT_WAVES, bool GATHERED>
__global__ void __launch_bounds__(kBlock) stage1_kernel(Stage1Args a) {
  using G = TileGeom<D>;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int kvh = blockIdx.y;
  char* my_lds = smem + wave * G::kBytes;

  if constexpr (!SPLIT_WAVES) {
    const int local = blockIdx.x * kWavesPerBlock + wave;
    if (local >= a.vnode_count) return;
    const VnodeView vn = load_vnode<GATHERED>(a, a.vnode_begin + local);
    const int rows_total = vn.q_len * a.g;
    for (int row0 = 0; row0 < rows_total; row0 += 16 * NQB) {
      WaveState<D, NQB> st;
      wave_attend<E, D, NQB, GATHERED>(a, vn, kvh, row0, 0, 1, my_lds, st);
      write_partials<D, NQB>(a, vn, kvh, row0, st);
    }
  } else {
    const VnodeView vn = load_vnode<GATHERED>(a, a.vnode_begin + blockIdx.x);
    const int rows_total = vn.q_len * a.g;
    for (int row0 = 0; row0 < rows_total; row0 += 16 * NQB) {
      WaveState<D, NQB> st;
      wave_attend<E, D, NQB, GATHERED>(a, vn, kvh, row0, wave, kWavesPerBlock, my_lds, st);
      merge_waves<D, NQB>(reinterpret_cast<float*>(smem), st);
      if (wave == 0) write_partials<D, NQB>(a, vn, kvh, row0, st);
      __syncthreads();  // staging LDS is reused by the next row chunk
    }
  }
}

// ---------------------------------------------------------------------------------------
// Wide vnodes: 32x32x16 MFMA tiles (twice the rate of 16x16x32 on this part), four waves per
// block with 32 query rows each and two blocks per compute unit, so that two waves share a SIMD
// and one wave's waits are filled by the other's instructions.  (Within a wave a tile step is one
// dependent chain, scores -> soft-max -> P.V; the matrix instructions of one wave overlap the
// vector instructions of the other about half of the time.)
// ---------------------------------------------------------------------------------------
constexpr int kWideWaves = 4;
constexpr int kWideBlock = kWave * kWideWaves;
constexpr int kWideRows = 32 * kWideWaves;        // query rows one pass of a block serves
constexpr int kWaveSlotsPerCu = 8;                // waves of these kernels a compute unit holds

// LDS layout of the wide kernel: rows of 2*D bytes back to back (no padding), 64-token super
// tiles of two 32-token tiles, a ring of kBufs buffers, then a staging area for the run's slot
// indices.  A row's 16-byte chunks are stored XOR-permuted: chunk c of row r sits in slot
// c ^ swz(r).  swz swaps the two low bit pairs of r, which makes both read patterns conflict free
// for 256-byte rows: the K operand read (16 different rows, same chunk) and the transposed V
// read (4 consecutive rows x 4 consecutive chunks).  Loads go global -> LDS directly; one wave
// instruction fills a 1 KB group of consecutive rows.
template <int D> struct WideGeom {
  static constexpr int kRowBytes = 2 * D;
  static constexpr int kChunks = D / 8;                  // 16-byte chunks per row
  static constexpr int kSub = 2;
  static constexpr int kTokens = kSub * kTileTokens;     // 64
  static constexpr int kBufs = 2;
  static constexpr int kAhead = kBufs - 1;               // super tiles in flight beyond the current one
  static constexpr int kTileBytes = kTileTokens * kRowBytes;
  static constexpr int kBytesK = kTokens * kRowBytes;
  static constexpr int kBytes = 2 * kBytesK;             // K + V of one buffer
  static constexpr int kRing = kBufs * kBytes;
  static constexpr int kGroupRows = kWave / kChunks;     // rows per 1 KB load group
  static constexpr int kGroups = kTokens / kGroupRows;   // groups per matrix and super tile
  static constexpr int kUnits = 2 * kGroups / kWideWaves;                       // loads per wave and super tile
  static constexpr int kSlots = kGroups >= kWideWaves ? kGroups / kWideWaves : 1;  // distinct rows among them
  static constexpr int kIdxCap = 2048;                    // slot indices staged at a time (tokens)
  static constexpr int kRecord = kRing + 4 * kIdxCap;    // byte offset of the program's record (kProgRecord ints)
  static constexpr int kLds = kRecord + 1024;
  static __device__ __forceinline__ int swz(int row) { return (((row & 3) << 2) | ((row >> 2) & 3)) & (kChunks - 1); }
};

// State of one wave for its 32 query rows.  o[db][j] = O[row lane%32][dim 32*db + 8*(j/4) +
// 4*(lane/32) + j%4]; m = soft-max reference (scaled scores, log2 domain); l = this lane's own
// share of the row sum until finish_state().
template <int D> struct WideState {
  f32x16 o[D / 32];
  float m;
  float l;
};

template <int D>
__device__ __forceinline__ void reset_state(WideState<D>& st) {
  st.m = -INFINITY;
  st.l = 0.f;
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int j = 0; j < 16; ++j) st.o[db][j] = 0.f;
}

// Query fragments of a wave's 32 rows, loaded in two steps so that other loads can be put
// between the two dependent ones: the address of a lane's row (needs the request id of the row,
// one load), then the fragments.  qf[ks]: row row0 + lane%32, dims 16*ks + 8*(lane/32) .. +7;
// zero past the vnode (src == nullptr).
// The record of a block program (kProgRecord ints, one thread of the block each): entries 0..3 are
// kv_off, kv_len, q_off and q_len of the program's first wide vnode, entry 4 says whether the rest is
// there (the vnode exists and has at most kWideRows query rows), entries kProgRecRequests.. the
// requests of its scratch rows, entries kProgRecSlots.. the pool slots of its first 64 tokens (the
// last token repeated past the end of a shorter run).  With it a block knows after one memory round
// trip what it otherwise learns in three (its table entry, the vnode's list entries, the request
// and slot lists) before it can ask for query and K/V rows.
constexpr int kProgRecord = 256;
constexpr int kProgRecRequests = 8;
constexpr int kProgRecSlots = kProgRecRequests + 128;
static_assert(kProgRecSlots + 64 <= kProgRecord && kProgRecord == 4 * 64, "one entry per thread of a block");

// (requests: the record's request entries in LDS, or null: the request of a row is read from the list)
template <bool GATHERED>
__device__ __forceinline__ const char* q_row_address32(const Stage1Args& a, const VnodeView& vn, int kvh, int row0,
                                                       const int* requests = nullptr) {
  const int lane = threadIdx.x & 63;
  const int r = row0 + (lane & 31), h = lane >> 5;
  if (r >= vn.q_len * a.g) return nullptr;
  const int ri = r / a.g;
  const int rj = r - ri * a.g;
  const int64_t entry = GATHERED ? (int64_t)(vn.q_off / a.nsplit)
                                 : (int64_t)(requests ? requests[ri] : a.q_entries[vn.q_off + ri]);
  return a.q + 2 * (entry * a.sq0 + (int64_t)(kvh * a.g + rj) * a.sq1 + 8 * h);
}
template <int D>
__device__ __forceinline__ void load_q_frags32(const char* src, u32x4 (&qf)[D / 16]) {
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
    u32x4 z = {0u, 0u, 0u, 0u};
    qf[ks] = src ? *reinterpret_cast<const u32x4*>(src + 32 * ks) : z;
  }
}

// Per-lane LDS byte addresses of the operand reads inside tile 0 of the current buffer, for
// contraction step / dim block 0.  Thanks to the XOR layout the address for step ks (dim block
// db) is the base with 32*ks (64*db) XOR-ed in; the second tile of the super tile is a constant
// offset away and buffer b of the ring is b * kBytes further (the ring starts on a multiple of the
// row size).
struct WideLane {
  unsigned k;     // K operand: row lane%32, chunk lane/32 (step ks: chunk 2*ks + lane/32)
  unsigned v_lo;  // transposed V read: tokens 4*(lane/32) + 0..3 (+16 for u = 1), dims 0..31
  unsigned v_hi;  // same, tokens + 8
};

template <int D>
__device__ __forceinline__ void init_lane(WideLane& la, unsigned ring) {
  using W = WideGeom<D>;
  const int lane = threadIdx.x & 63;
  const int p32 = lane & 31, h = lane >> 5, p = lane & 15, gi = (lane >> 4) & 1;
  la.k = ring + p32 * W::kRowBytes + 16 * ((h & (W::kChunks - 1)) ^ W::swz(p32));
  const int row_lo = 4 * h + (p >> 2), row_hi = row_lo + 8;
  const int chunk = (2 * gi + ((p & 3) >> 1)) & (W::kChunks - 1);
  la.v_lo = ring + W::kBytesK + row_lo * W::kRowBytes + 16 * (chunk ^ W::swz(row_lo)) + 8 * (p & 1);
  la.v_hi = ring + W::kBytesK + row_hi * W::kRowBytes + 16 * (chunk ^ W::swz(row_hi)) + 8 * (p & 1);
}

// Byte offset of an object of the block's dynamic LDS segment within LDS.
__device__ __forceinline__ unsigned lds_offset(const void* p) {
  return (unsigned)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}

__device__ __forceinline__ WideLane at_buffer(const WideLane& la0, unsigned buffer_offset) {
  return WideLane{la0.k + buffer_offset, la0.v_lo + buffer_offset, la0.v_hi + buffer_offset};
}

// 16 bytes per lane from global memory straight into LDS at lds_base + 16 * lane (lds_base is
// wave uniform).  Written as assembly on purpose: for the builtin the compiler cannot tell which
// later LDS reads touch the landing bytes and makes every one of them wait for all such loads
// in flight, which serialises the stream with the arithmetic.  Completion is awaited by hand
// with wait_direct_loads<N>() before the block barrier that publishes a buffer.
__device__ __forceinline__ void load_direct16(const char* src, unsigned lds_base) {
  // (M0 holds the LDS address: bound as an operand, so the compiler writes it and knows it is live)
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "{m0}"(lds_base) : "memory");
}
// Wait until at most N of this wave's vector-memory operations are still in flight (they finish
// in order).
template <int N>
__device__ __forceinline__ void wait_direct_loads() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ u32x4 lds_read16(unsigned addr) {
  return *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>((uintptr_t)addr);
}
__device__ __forceinline__ u32x2 lds_read_tr8(unsigned addr) {
  const i16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      reinterpret_cast<__attribute__((address_space(3))) i16x4*>((uintptr_t)addr));
  return __builtin_bit_cast(u32x2, v);
}

// The soft-max reference m of a row is updated lazily: only when the row's running maximum
// exceeds it by more than kSlack (log2 units).  Probabilities therefore stay below 2^kSlack --
// exact in any case, since numerator and denominator share the reference -- and the
// accumulators are rescaled rarely (in practice once, on a run's first tile).
constexpr float kSlack = 8.f;

// A tile step without a per-query mask (every row of the vnode attends every token of the run).
struct NoMask {
  __device__ __forceinline__ void operator()(f32x16&) const {}
};

// One 32-token step for the wave's 32 rows on the tile `off` bytes into the current buffer.
// S^T = K Q^T: A = K rows (token lane%32, 8 dims per lane), B = Q; accumulator register j of a
// lane is token 8*(j/4) + 4*(lane/32) + j%4.  Registers 8u .. 8u+7 are exactly the 8 k-slots a
// lane feeds to the u-th P.V contraction, whose A operand (V^T) comes from two transposed LDS
// reads of 4 consecutive tokens each.  valid < 32 only on a run's last, partial tile.  `mask`
// is applied to the raw scores (it overwrites those of tokens the lane's row does not attend).
template <typename E, int D, typename Mask = NoMask>
__device__ __forceinline__ void tile_step32(const WideLane& la, unsigned off, int valid, float sc,
                                            const u32x4 (&qf)[D / 16], WideState<D>& st, const Mask& mask = Mask()) {
  using W = WideGeom<D>;
  constexpr int KS = D / 16, DB = D / 32, NV = 2 * DB;

  // the K operands are requested eight contraction steps at a time, before the first of those
  // steps needs one (all of them at once up to head_dim 128)
  const unsigned kb = la.k + off;
  constexpr int KB = KS < 8 ? KS : 8;
  f32x16 s;
#pragma unroll
  for (int j = 0; j < 16; ++j) s[j] = 0.f;
#pragma unroll
  for (int k0 = 0; k0 < KS; k0 += KB) {
    u32x4 kf[KB];
#pragma unroll
    for (int ks = 0; ks < KB; ++ks) kf[ks] = lds_read16(kb ^ (32u * (k0 + ks)));
    // (keeps the scheduler from sinking each read next to its use, which would expose the full
    // LDS latency eight times in a row)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < KB; ++ks) s = E::mfma32(kf[ks], qf[k0 + ks], s);
  }

  if (valid < kTileTokens) {  // wave uniform
    asm volatile("" ::: "memory");  // keeps this a branch: as selects it would run on every tile
    const int h = (threadIdx.x & 63) >> 5;
#pragma unroll
    for (int j = 0; j < 16; ++j) s[j] = (8 * (j >> 2) + 4 * h + (j & 3) >= valid) ? -INFINITY : s[j];
  }
  mask(s);

  // the V^T operands do not depend on the probabilities: request them now, so that they arrive
  // under the soft-max arithmetic (they take the registers the K operands just left); at
  // head_dim 256 only those of the first 16 tokens, the others after the first half of P.V
  const unsigned vlo = la.v_lo + off, vhi = la.v_hi + off;
  constexpr int VH = D > 128 ? DB : NV;   // operands requested ahead of the soft-max
  u32x4 vf[VH];
  auto read_v = [&](int i) {
    const int u = i / DB, db = i % DB;
    const u32x2 lo = lds_read_tr8((vlo ^ (64u * db)) + u * 16 * W::kRowBytes);
    const u32x2 hi = lds_read_tr8((vhi ^ (64u * db)) + u * 16 * W::kRowBytes);
    return u32x4{lo[0], lo[1], hi[0], hi[1]};
  };
#pragma unroll
  for (int i = 0; i < VH; ++i) vf[i] = read_v(i);
  __builtin_amdgcn_sched_barrier(0);
  float mx = max3(s[0], s[1], s[2]);
#pragma unroll
  for (int j = 3; j < 15; j += 2) mx = max3(mx, s[j], s[j + 1]);
  mx = xor32_max(fmaxf(mx, s[15])) * sc;  // sc > 0; finite: the tile holds at least one token
  const bool grow = mx > st.m + kSlack;   // also true on a run's first tile (m = -inf)
  if (__builtin_amdgcn_ballot_w64(grow)) {
    const float m_new = grow ? mx : st.m;
    const float alpha = __builtin_amdgcn_exp2f(st.m - m_new);
    st.l *= alpha;
#pragma unroll
    for (int db = 0; db < DB; ++db) st.o[db] *= alpha;
    st.m = m_new;
  }

  const float neg_m = -st.m;
  float x[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) x[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[j], sc, neg_m));
  u32x4 pf[2];
#pragma unroll
  for (int u = 0; u < 2; ++u)
    pf[u] = u32x4{E::pack2(x[8 * u + 0], x[8 * u + 1]), E::pack2(x[8 * u + 2], x[8 * u + 3]),
                  E::pack2(x[8 * u + 4], x[8 * u + 5]), E::pack2(x[8 * u + 6], x[8 * u + 7])};
  // the row sum is taken over the probabilities as P.V will see them (rounded to the storage
  // type), two per instruction
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int i = 0; i < 4; ++i) st.l = E::add_pair(pf[u][i], st.l);

#pragma unroll
  for (int i = 0; i < VH; ++i) st.o[i % DB] = E::mfma32(vf[i], pf[i / DB], st.o[i % DB]);
  if constexpr (VH < NV) {
    u32x4 vg[NV - VH];
#pragma unroll
    for (int i = VH; i < NV; ++i) vg[i - VH] = read_v(i);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = VH; i < NV; ++i) st.o[i % DB] = E::mfma32(vg[i - VH], pf[i / DB], st.o[i % DB]);
  }
}

template <int D>
__device__ __forceinline__ void finish_state(WideState<D>& st) {
  st.l = xor32_sum(st.l);
}

// (ROUND16: the normalised output is rounded to fp16 on its way to the fp32 scratch)
template <int D, bool ROUND16 = false>
__device__ __forceinline__ void write_partials32(const Stage1Args& a, const VnodeView& vn, int kvh, int row0,
                                                 const WideState<D>& st) {
  const int lane = threadIdx.x & 63;
  const int r = row0 + (lane & 31), h = lane >> 5;
  if (r >= vn.q_len * a.g) return;
  const int ri = r / a.g, rj = r - ri * a.g;
  const int64_t row = vn.q_off + ri;
  const int head = kvh * a.g + rj;
  const float inv = st.l > 0.f ? 1.f / st.l : 0.f;
  float* dst = a.mid_o + row * a.so0 + (int64_t)head * a.so1 + 4 * h;
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      f32x4 v = {st.o[db][4 * jj] * inv, st.o[db][4 * jj + 1] * inv, st.o[db][4 * jj + 2] * inv,
                 st.o[db][4 * jj + 3] * inv};
      if constexpr (ROUND16) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (float)(_Float16)v[e];
      }
      *reinterpret_cast<f32x4*>(dst + 32 * db + 8 * jj) = v;
    }
  if (h == 0) a.mid_lse[row * a.sl0 + head] = st.l > 0.f ? (__builtin_amdgcn_logf(st.l) + st.m) * kLn2 : -INFINITY;
}

// Merge of the TG waves that hold the same rows (token groups 0..TG-1 of row group rg) into
// token group 0, pairwise through LDS.  Every wave of the block must call this.
template <int D>
__device__ __forceinline__ void merge_token_groups(float* xchg, WideState<D>& st, int rg, int tg, int tgroups, bool active) {
  constexpr int NV = (D / 32) * 16 + 2;
  const int lane = threadIdx.x & 63;
  for (int half = tgroups >> 1; half >= 1; half >>= 1) {
    __syncthreads();
    if (active && tg >= half && tg < 2 * half) {
      float* dst = xchg + (size_t)(rg * half + tg - half) * NV * kWave + lane;
      int n = 0;
      dst[(n++) * kWave] = st.m;
      dst[(n++) * kWave] = st.l;
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int j = 0; j < 16; ++j) dst[(n++) * kWave] = st.o[db][j];
    }
    __syncthreads();
    if (active && tg < half) {
      const float* src = xchg + (size_t)(rg * half + tg) * NV * kWave + lane;
      int n = 0;
      const float m2 = src[(n++) * kWave];
      const float l2 = src[(n++) * kWave];
      const float m = fmaxf(st.m, m2);
      const float a1 = scale_from(st.m, m), a2 = scale_from(m2, m);
      st.l = st.l * a1 + l2 * a2;
      st.m = m;
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int j = 0; j < 16; ++j) st.o[db][j] = st.o[db][j] * a1 + src[(n++) * kWave] * a2;
    }
  }
}

// One block (kWideWaves waves) serves the row pieces chunk, chunk + chunks, ... (kWideRows query
// rows each) of a vnode for one kv head.  The block
// streams the vnode's KV run through a ring of kBufs 64-token LDS buffers with direct
// global->LDS loads, kBufs - 1 super tiles ahead of the one being consumed; the run's slot
// indices are staged in LDS first so that nothing but those loads is in flight in the loop.
// Per pass over the run the waves form RG row groups of 32 query rows x TG token groups
// (RG * TG = kWideWaves): a wave consumes the 32-token tiles t with t % TG == tg for the rows of
// its row group, and the TG states of a row group are merged at the end.
template <typename E, int D, bool GATHERED>
__device__ __forceinline__ void wide_block(const Stage1Args& a, char* smem, const VnodeView& vn, int kvh, int chunk,
                                           int chunks, const int* record = nullptr) {
  using W = WideGeom<D>;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int rows_total = vn.q_len * a.g;
  const int nsuper = (vn.kv_len + W::kTokens - 1) / W::kTokens;

  // loader role of this lane: 16-byte slot `pos` of row `grp_row` in each 1 KB group it fills
  const int grp_row = lane / W::kChunks, pos = lane % W::kChunks;
  const char* kbase = a.k + 2 * ((int64_t)kvh * a.sk1);
  const char* vbase = a.v + 2 * ((int64_t)kvh * a.sv1);
  const unsigned k_stride = (unsigned)(2 * a.sk0), v_stride = (unsigned)(2 * a.sv0);  // bytes, < 2^32 (checked by the host)
  int* idx_lds = reinterpret_cast<int*>(smem + W::kRing);
  const unsigned ring = lds_offset(smem);

  // this block's pieces of kWideRows rows: chunk, chunk + chunks, ...
  for (int piece = chunk; piece * kWideRows < rows_total; piece += chunks) {
  const int rows_end = min((piece + 1) * kWideRows, rows_total);
  for (int row0 = piece * kWideRows; row0 < rows_end;) {
    // waves as rgroups row groups x tgroups token groups: halve the row groups (down to a token
    // split of four) while the rows left in the piece leave half of them without rows
    const int groups = (rows_end - row0 + 31) >> 5;   // 32-row groups still to serve
    int rgroups = kWideWaves, tgroups = 1;
    while (tgroups < 4 && 2 * groups <= rgroups) {
      rgroups >>= 1;
      tgroups <<= 1;
    }
    const int rg = wave / tgroups, tg = wave % tgroups;
    const int my_row0 = row0 + 32 * rg;
    const bool active = rg < rgroups && my_row0 < rows_end;

    // start-up chain: [request ids of the rows, slot indices] -> [Q fragments, first K/V rows]
    // (the program's record covers the vnode's first kWideRows rows: its first piece, one pass)
    // (not at head_dim 256, where the step has no register to spare)
    const int* rec = (!GATHERED && D <= 128 && piece == 0) ? record : nullptr;   // block uniform
    const char* q_src = q_row_address32<GATHERED>(a, vn, kvh, active ? my_row0 : rows_total,
                                                  rec ? rec + kProgRecRequests : nullptr);
    u32x4 qf[D / 16];
    WideState<D> st;
    reset_state<D>(st);
    WideLane la0;
    init_lane<D>(la0, ring);
    unsigned cur = 0;  // byte offset of the ring buffer that holds the current super tile

    // slot indices of tokens [idx_base, idx_base + kIdxCap) of the run, staged by the whole block
    int idx_base = 0;
    auto stage_indices = [&](int base) {
      if constexpr (!GATHERED) {
        idx_base = base;
        // (branch free, so that the loads are in flight together; entries past the run repeat its last)
        int e[W::kIdxCap / kWideBlock];
#pragma unroll
        for (int i = 0; i < W::kIdxCap / kWideBlock; ++i)
          e[i] = a.kv_entries[vn.kv_base + min(base + kWideBlock * i + (int)threadIdx.x, vn.kv_len - 1)];
#pragma unroll
        for (int i = 0; i < W::kIdxCap / kWideBlock; ++i) idx_lds[kWideBlock * i + threadIdx.x] = e[i];
        __syncthreads();
      }
    };
    // rows of super tile j -> ring buffer j % kBufs, in two steps: read_rows(j) takes the slot
    // indices of the rows this wave loads out of LDS (one super tile ahead of the loads, so that
    // the LDS round trip is hidden by a tile step), issue_rows(j) requests the rows.  Tokens past
    // the run repeat its last token: the scores of such rows are masked and their V rows are finite.
    unsigned srow[W::kSlots];
    auto read_rows = [&](int j) {
      if (j >= nsuper) return;
      if constexpr (!GATHERED) {
        if (j * W::kTokens >= idx_base + W::kIdxCap) {  // block uniform
          __syncthreads();                              // every wave has read the indices it needed
          stage_indices(idx_base + W::kIdxCap);
        }
      }
#pragma unroll
      for (int u = 0; u < W::kSlots; ++u) {
        const int grp = W::kGroups >= kWideWaves ? u * kWideWaves + wave : wave % W::kGroups;
        const int row = grp * W::kGroupRows + grp_row;
        const int t = min(j * W::kTokens + row, vn.kv_len - 1);
        srow[u] = GATHERED ? (unsigned)(vn.kv_base + t) : (unsigned)idx_lds[t - idx_base];
      }
    };
    auto issue_rows = [&](int j) {
      if (j >= nsuper) return;
      const unsigned buf = ring + (unsigned)(j % W::kBufs) * W::kBytes;
#pragma unroll
      for (int u = 0; u < W::kUnits; ++u) {
        // unit u of this wave: K groups first, then V groups
        const bool is_v = W::kGroups >= kWideWaves ? u >= W::kSlots : wave >= W::kGroups;
        const int sl = u % W::kSlots;
        const int grp = W::kGroups >= kWideWaves ? sl * kWideWaves + wave : wave % W::kGroups;
        const int row = grp * W::kGroupRows + grp_row;
        const char* src = (is_v ? vbase : kbase) + (uint64_t)srow[sl] * (is_v ? v_stride : k_stride);
        load_direct16(src + 16 * (pos ^ W::swz(row)), buf + (is_v ? W::kBytesK : 0) + grp * 1024);
      }
    };
    static_assert(W::kAhead == 1, "the record path below requests exactly the first super tile");
    if (rec && nsuper > 0) {
      // the first super tile's slots come with the record: its rows are requested before the
      // run's index list has been read at all
#pragma unroll
      for (int u = 0; u < W::kSlots; ++u) {
        const int grp = W::kGroups >= kWideWaves ? u * kWideWaves + wave : wave % W::kGroups;
        srow[u] = (unsigned)rec[kProgRecSlots + grp * W::kGroupRows + grp_row];
      }
      issue_rows(0);
      stage_indices(0);
    } else {
      if (nsuper > 0) stage_indices(0);  // block uniform
#pragma unroll
      for (int j = 0; j < W::kAhead; ++j) {
        read_rows(j);
        issue_rows(j);
      }
    }
    read_rows(W::kAhead);
    load_q_frags32<D>(q_src, qf);
    // nothing the compiler itself tracks (the Q fragments) may still be in flight in the loop:
    // a wait for it there would also wait for every direct load
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    // (and the compiler must see the fragments as complete, or it keeps a wait for them in the loop)
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) asm volatile("" : "+v"(qf[ks]));
    for (int super = 0; super < nsuper; ++super) {
      // publish super tile `super` to the block; the ones after it may stay in flight
      const int behind = min(nsuper - 1 - super, W::kAhead - 1);
      if (behind >= 2) wait_direct_loads<2 * W::kUnits>();
      else if (behind == 1) wait_direct_loads<W::kUnits>();
      else wait_direct_loads<0>();
      __syncthreads();
      // the buffer consumed before that barrier is free: refill it
      issue_rows(super + W::kAhead);
      read_rows(super + W::kAhead + 1);
      if (active) {
        const WideLane la = at_buffer(la0, cur);
#pragma unroll 1
        for (int sub = 0; sub < W::kSub; ++sub) {
          const int tile = super * W::kSub + sub;
          if ((tile & (tgroups - 1)) != tg) continue;
          const int valid = vn.kv_len - tile * kTileTokens;
          if (valid > 0) tile_step32<E, D>(la, sub * W::kTileBytes, valid, a.scale_log2, qf, st);
        }
      }
      cur = cur + W::kBytes == W::kRing ? 0u : cur + W::kBytes;
    }
    finish_state<D>(st);
    if (tgroups > 1) merge_token_groups<D>(reinterpret_cast<float*>(smem), st, rg, tg, tgroups, active);
    if (active && tg == 0) write_partials32<D>(a, vn, kvh, my_row0, st);
    __syncthreads();  // staging LDS is reused by the next pass over the run
    row0 += 32 * rgroups;
  }
  }
}

// ---------------------------------------------------------------------------------------
// Narrow vnodes (at most 16 query rows): one wave per (vnode, kv head) streams the run through
// a wave-private LDS tile of 32 tokens with direct global->LDS loads, in the same unpadded XOR
// layout as the wide kernel.  K and V have one tile each: the K rows of the next tile are
// requested as soon as the scores of the current one are out of LDS, its V rows as soon as the
// current P.V is, so a leaf vnode of a few dozen tokens costs little more than its two memory
// round trips (slot indices, rows).  Slot indices are staged 256 tokens at a time.
// ---------------------------------------------------------------------------------------
template <int D> struct NarrowGeom {
  static constexpr int kRowBytes = 2 * D;
  static constexpr int kChunks = D / 8;
  static constexpr int kBytesK = kTileTokens * kRowBytes;
  static constexpr int kBytes = 2 * kBytesK;
  static constexpr int kGroupRows = kWave / kChunks;            // rows per 1 KB load
  static constexpr int kGroups = kTileTokens / kGroupRows;      // loads per matrix and tile
  static constexpr int kIdxCap = 256;
  static constexpr int kLds = kBytes + 4 * kIdxCap;             // per wave; a multiple of the row size
  static __device__ __forceinline__ int swz(int row) { return (((row & 3) << 2) | ((row >> 2) & 3)) & (kChunks - 1); }
};

// Layout of a narrow vnode's record in Stage1Args::narrow_table (ints): kv_off, kv_len, q_off,
// q_len; then the requests of the vnode's first kNarrowRecRequests scratch rows; then the pool slots
// of its first kTileTokens tokens (the last one repeated past the end of a shorter run).
constexpr int kNarrowRecord = 64;
constexpr int kNarrowRecRequests = 16;
constexpr int kNarrowRecSlots = 4 + kNarrowRecRequests;

// One wave's share of a narrow vnode for the 16 query rows from row0: the tiles tile0,
// tile0 + tstride, ... of the run, staged in the wave's own LDS area at lds0.  `rec` is the lane's
// int of the vnode's record when `inlined` (else unused).
template <typename E, int D, bool GATHERED>
__device__ __forceinline__ void narrow_attend(const Stage1Args& a, const VnodeView& vn, char* smem, unsigned lds0,
                                              int kvh, int row0, int tile0, int tstride, WaveState<D, 1>& st,
                                              int rec = 0, bool inlined = false) {
  using N = NarrowGeom<D>;
  constexpr int KS = D / 32, DB = D / 16;
  constexpr float kSlackN = 8.f;
  const int lane = threadIdx.x & 63;
  const int p = lane & 15, c = lane >> 4;
  const int ntiles = (vn.kv_len + kTileTokens - 1) / kTileTokens;
  int* idx_lds = reinterpret_cast<int*>(smem + lds0 + N::kBytes);
  const unsigned tile0_addr = lds_offset(smem) + lds0;  // the wave's K tile; its V tile follows

  // loader role: 16-byte slot `pos` of row `grp_row` in each 1 KB group
  const int grp_row = lane / N::kChunks, pos = lane % N::kChunks;
  const char* kbase = a.k + 2 * ((int64_t)kvh * a.sk1);
  const char* vbase = a.v + 2 * ((int64_t)kvh * a.sv1);
  const unsigned k_stride = (unsigned)(2 * a.sk0), v_stride = (unsigned)(2 * a.sv0);  // bytes, < 2^32 (checked by the host)

  // operand read addresses: K row 16*tb + p, chunk c (contraction step ks: chunk 4*ks + c);
  // V tokens 4*c + p/4 (+16), chunk 2*db + (p%4)/2, half p%2
  unsigned k_addr[2], v_addr[2];
#pragma unroll
  for (int tb = 0; tb < 2; ++tb) {
    const int kr = 16 * tb + p, vr = 16 * tb + 4 * c + (p >> 2);
    k_addr[tb] = tile0_addr + kr * N::kRowBytes + 16 * ((c & (N::kChunks - 1)) ^ N::swz(kr));
    v_addr[tb] = tile0_addr + N::kBytesK + vr * N::kRowBytes + 16 * ((((p & 3) >> 1) & (N::kChunks - 1)) ^ N::swz(vr)) + 8 * (p & 1);
  }

  // start-up chain: [request id of the lane's row, slot indices] -> [Q fragments, first K/V rows].
  // Fragment ks of a lane: row row0 + p, dims 32*ks + 8*c .. +7; zero past the vnode.
  const char* q_src = nullptr;
  {
    const int r = min(row0 + p, max(vn.q_len * a.g - 1, 0)), ri = r / a.g, rj = r - ri * a.g;
    // (the record holds the requests of the first rows; every lane takes part in the exchange)
    const bool from_record = inlined && vn.q_len <= kNarrowRecRequests;
    const int listed = from_record ? __shfl(rec, 4 + ri) : 0;
    if (row0 + p < vn.q_len * a.g) {
      const int64_t entry = GATHERED ? (int64_t)(vn.q_off / a.nsplit)
                                     : (from_record ? (int64_t)listed : (int64_t)a.q_entries[vn.q_off + ri]);
      q_src = a.q + 2 * (entry * a.sq0 + (int64_t)(kvh * a.g + rj) * a.sq1 + 8 * c);
    }
  }
  u32x4 qf[1][KS];
  reset_state<D, 1>(st);
  if (tile0 < ntiles) {
    // slot indices of tokens [idx_base, idx_base + kIdxCap) of the run
    int idx_base = 0;
    auto stage_indices = [&](int base) {
      if constexpr (!GATHERED) {
        idx_base = base;
        // (branch free, so that the loads are in flight together; entries past the run repeat its last)
        int e[N::kIdxCap / kWave];
#pragma unroll
        for (int i = 0; i < N::kIdxCap / kWave; ++i)
          e[i] = a.kv_entries[vn.kv_base + min(base + kWave * i + lane, vn.kv_len - 1)];
#pragma unroll
        for (int i = 0; i < N::kIdxCap / kWave; ++i) idx_lds[kWave * i + lane] = e[i];
        wave_lds_fence();
      }
    };
    // K (or V) rows of `tile` -> the wave's K (V) tile.  Tokens past the run repeat its last
    // token (their scores are masked, their V rows are finite).  The slot indices are read
    // from the staged window each time rather than kept in registers between the two calls.
    auto issue = [&](int tile, bool is_v) {
      if constexpr (!GATHERED) {
        if (tile * kTileTokens >= idx_base + N::kIdxCap) stage_indices(tile * kTileTokens);
      }
      // (all index reads first: a load instruction is a fence for the compiler, so reads placed
      // between the loads would each be waited for on its own)
      unsigned srow[N::kGroups];
#pragma unroll
      for (int g = 0; g < N::kGroups; ++g) {
        const int t = min(tile * kTileTokens + g * N::kGroupRows + grp_row, vn.kv_len - 1);
        srow[g] = GATHERED ? (unsigned)(vn.kv_base + t) : (unsigned)idx_lds[t - idx_base];
      }
#pragma unroll
      for (int g = 0; g < N::kGroups; ++g) {
        const int row = g * N::kGroupRows + grp_row;
        const char* src = (is_v ? vbase : kbase) + (uint64_t)srow[g] * (is_v ? v_stride : k_stride) + 16 * (pos ^ N::swz(row));
        load_direct16(src, tile0_addr + (is_v ? N::kBytesK : 0) + g * 1024);
      }
    };
    // With the vnode's record at hand and the run's first tile to serve, the first 32 slot
    // indices are already here: the rows are requested at once, and the rest of the window (if
    // the run is longer than a tile) arrives beside them.
    const bool from_record = !GATHERED && inlined && tile0 == 0;
    int rest[N::kIdxCap / kWave];
    if (from_record) {
      if (lane >= kNarrowRecSlots && lane < kNarrowRecSlots + kTileTokens) idx_lds[lane - kNarrowRecSlots] = rec;
      wave_lds_fence();
      idx_base = 0;
      issue(0, false);
      issue(0, true);
      if (vn.kv_len > kTileTokens) {
#pragma unroll
        for (int i = 0; i < N::kIdxCap / kWave; ++i)
          rest[i] = a.kv_entries[vn.kv_base + min(kWave * i + lane, vn.kv_len - 1)];
      }
    } else {
      stage_indices(tile0 * kTileTokens);
      issue(tile0, false);
      issue(tile0, true);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 z = {0u, 0u, 0u, 0u};
      qf[0][ks] = q_src ? *reinterpret_cast<const u32x4*>(q_src + 64 * ks) : z;
    }
    // nothing the compiler itself tracks may still be in flight below: a wait for it would
    // also wait for every direct load
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    if (from_record && vn.kv_len > kTileTokens) {
      // (the first tile's rows were requested with the record's indices, which these repeat)
#pragma unroll
      for (int i = 0; i < N::kIdxCap / kWave; ++i) idx_lds[kWave * i + lane] = rest[i];
      wave_lds_fence();
    }
    // (and the compiler must see the fragments as complete, or it keeps a wait for them in the loop)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(qf[0][ks]));
    for (int tile = tile0; tile < ntiles; tile += tstride) {
      const int next = tile + tstride;
      const bool more = next < ntiles;
      const int valid = vn.kv_len - tile * kTileTokens;
      // ---- S^T = K Q^T : s[tb][j] = score(token 16*tb + 4*c + j, row p)
      wait_direct_loads<N::kGroups>();  // K landed; V may still be in flight
      f32x4 s[2];
#pragma unroll
      for (int tb = 0; tb < 2; ++tb) {
        s[tb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s[tb] = E::mfma(lds_read16(k_addr[tb] ^ (64u * ks)), qf[0][ks], s[tb]);
      }
      if (more) {
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the K tile has been read
        issue(next, false);
      }
      if (valid < kTileTokens) {
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (16 * tb + 4 * c + j >= valid) s[tb][j] = -INFINITY;
      }
      // online soft-max with a lazily updated reference (see tile_step)
      float mx = fmaxf(fmaxf(fmaxf(s[0][0], s[0][1]), fmaxf(s[0][2], s[0][3])),
                       fmaxf(fmaxf(s[1][0], s[1][1]), fmaxf(s[1][2], s[1][3])));
      mx = xor32_max(xor16_max(mx)) * a.scale_log2;
      const bool grow = mx > st.m[0] + kSlackN;
      if (__builtin_amdgcn_ballot_w64(grow)) {
        const float m_new = grow ? mx : st.m[0];
        const float alpha = __builtin_amdgcn_exp2f(st.m[0] - m_new);
        st.l[0] *= alpha;
#pragma unroll
        for (int db = 0; db < DB; ++db) st.o[0][db] *= alpha;
        st.m[0] = m_new;
      }
      const float neg_m = -st.m[0];
      float x[8];
      float sum = 0.f;
#pragma unroll
      for (int tb = 0; tb < 2; ++tb)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          x[4 * tb + j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[tb][j], a.scale_log2, neg_m));
          sum += x[4 * tb + j];
        }
      st.l[0] += sum;
      const u32x4 pf = {E::pack2(x[0], x[1]), E::pack2(x[2], x[3]), E::pack2(x[4], x[5]), E::pack2(x[6], x[7])};
      // ---- O^T += V^T P^T
      if (more) wait_direct_loads<N::kGroups>();  // V landed; the next K may be in flight
      else wait_direct_loads<0>();
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const u32x2 lo = lds_read_tr8(v_addr[0] ^ (32u * db));
        const u32x2 hi = lds_read_tr8(v_addr[1] ^ (32u * db));
        const u32x4 vf = {lo[0], lo[1], hi[0], hi[1]};
        st.o[0][db] = E::mfma(vf, pf, st.o[0][db]);
      }
      if (more) {
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the V tile has been read
        issue(next, true);
      }
    }
  }
  finish_state<D, 1>(st);
}

// Merge of the `share` waves of one narrow vnode (same rows, interleaved tiles) into the first of
// them, pairwise through LDS at xchg.  Every wave of the block calls this (block barriers).
template <int D>
__device__ __forceinline__ void merge_shares(float* xchg, WaveState<D, 1>& st, int w, int share) {
  constexpr int NV = (D / 16) * 4 + 2;  // floats of state per lane
  const int lane = threadIdx.x & 63;
  for (int half = share >> 1; half >= 1; half >>= 1) {
    __syncthreads();
    if (w >= half && w < 2 * half) {
      float* dst = xchg + (size_t)(w - half) * NV * kWave + lane;
      int n = 0;
      dst[(n++) * kWave] = st.m[0];
      dst[(n++) * kWave] = st.l[0];
#pragma unroll
      for (int db = 0; db < D / 16; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[(n++) * kWave] = st.o[0][db][j];
    }
    __syncthreads();
    if (w < half) {
      const float* src = xchg + (size_t)w * NV * kWave + lane;
      int n = 0;
      const float m2 = src[(n++) * kWave];
      const float l2 = src[(n++) * kWave];
      const float m = fmaxf(st.m[0], m2);
      const float a1 = scale_from(st.m[0], m), a2 = scale_from(m2, m);
      st.l[0] = st.l[0] * a1 + l2 * a2;
      st.m[0] = m;
#pragma unroll
      for (int db = 0; db < D / 16; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) st.o[0][db][j] = st.o[0][db][j] * a1 + src[(n++) * kWave] * a2;
    }
  }
}

// A narrow vnode served by `share` consecutive waves of a block (share = 1, 2 or 4, the same
// for the whole launch; the host picks more than one when there are fewer vnodes than wave
// slots): wave w of the vnode takes the tiles w, w + share, ..., and the shares are merged
// through LDS.  `slot` is the wave's index in the block; a wave without a vnode (exists ==
// false) only keeps the block's barriers company.
template <typename E, int D, bool GATHERED>
__device__ __forceinline__ void narrow_item(const Stage1Args& a, char* smem, int slot, int share, bool exists,
                                            int vnode, int kvh) {
  using N = NarrowGeom<D>;
  const unsigned lds0 = (unsigned)slot * N::kLds;  // byte offset of the wave's area in the block's LDS segment
  VnodeView vn{0, 0, 0, 0};
  int rec = 0;
  const bool inlined = !GATHERED && a.narrow_table != nullptr;   // launch uniform
  if (inlined) {
    if (exists) rec = a.narrow_table[(int64_t)(vnode - a.narrow_begin) * kNarrowRecord + (threadIdx.x & 63)];
    vn.kv_base = __builtin_amdgcn_readlane(rec, 0);
    vn.kv_len = __builtin_amdgcn_readlane(rec, 1);
    vn.q_off = __builtin_amdgcn_readlane(rec, 2);
    vn.q_len = __builtin_amdgcn_readlane(rec, 3);
  } else if (exists) {
    vn = load_vnode<GATHERED>(a, vnode);
  }
  const int rows_total = vn.q_len * a.g;
  if (share == 1) {
    for (int row0 = 0; row0 < rows_total; row0 += 16) {
      WaveState<D, 1> st;
      narrow_attend<E, D, GATHERED>(a, vn, smem, lds0, kvh, row0, 0, 1, st, rec, inlined);
      write_partials<D, 1>(a, vn, kvh, row0, st);
    }
    return;
  }
  const int w = slot & (share - 1);
  float* xchg = reinterpret_cast<float*>(smem + (size_t)(slot - w) * N::kLds);
  // every wave of the block makes the same number of passes (block barriers inside): the most
  // any of its vnodes needs, agreed on through one word of each wave's LDS area
  const int nwaves = blockDim.x >> 6;
  *reinterpret_cast<volatile int*>(smem + lds0) = (rows_total + 15) >> 4;
  __syncthreads();
  int passes = 0;
  for (int i = 0; i < nwaves; ++i) passes = max(passes, *reinterpret_cast<volatile int*>(smem + (size_t)i * N::kLds));
  __syncthreads();
  for (int pass = 0; pass < passes; ++pass) {
    const int row0 = 16 * pass;
    WaveState<D, 1> st;
    if (row0 < rows_total) narrow_attend<E, D, GATHERED>(a, vn, smem, lds0, kvh, row0, w, share, st, rec, inlined);
    else reset_state<D, 1>(st);
    merge_shares<D>(xchg, st, w, share);
    if (w == 0 && row0 < rows_total) write_partials<D, 1>(a, vn, kvh, row0, st);
    __syncthreads();  // the exchange area is the staging area of the next pass
  }
}

// Narrow vnodes alone (a launch without wide vnodes), one vnode per block of `narrow_share`
// waves: the footprint of one LDS tile per wave instead of a wide block's ring, so that more of
// these latency-bound waves share a compute unit.
template <typename E, int D, bool GATHERED>
__global__ void __launch_bounds__(kWideBlock) stage1_narrow_kernel(Stage1Args a) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int local_vnode = blockIdx.x / a.hkv;
  narrow_item<E, D, GATHERED>(a, smem, wave, a.narrow_share, true, a.narrow_begin + local_vnode,
                              blockIdx.x - local_vnode * a.hkv);
}

// Blocks are handed to compute units in index order as units become free, so serving the wide
// vnodes in order of decreasing work (query rows x tokens) is longest-job-first list scheduling:
// the machine does not end on a late start of a long block.  Every block ranks the wide vnodes
// itself (they are few) and takes the one whose rank is `target`.  Block uniform.
//
// On the way, neighbours in the vnode list that attend the same KV run with adjoining scratch
// rows -- the query tiles the planner cut one node into -- are joined into one work item of at
// most `cap` query rows (what the blocks of one vnode serve in a single pass): a tile of 16
// requests x 4 heads fills only half of a block's rows, and two such tiles would stage the same
// run twice.  The first vnode of a group carries the group; the others become empty items.
constexpr int kMaxRanked = kWideBlock;
template <bool GATHERED>
__device__ __forceinline__ int wide_vnode_of_rank(const Stage1Args& a, char* smem, int target, VnodeView& view) {
  const int n = a.vnode_count;
  if (n < 2 || n > kMaxRanked) {
    view = load_vnode<GATHERED>(a, a.vnode_begin + target);
    return target;
  }
  // keys[u]: work of vnode u in 23 bits (a float's exponent and leading mantissa bits), then
  // 256 - u: larger key = earlier, no two equal; 0 for a vnode that is not the head of a group
  unsigned* keys = reinterpret_cast<unsigned*>(smem);
  VnodeView* views = reinterpret_cast<VnodeView*>(keys + kMaxRanked);
  int* group_q_len = reinterpret_cast<int*>(views + kMaxRanked);
  unsigned long long* joined = reinterpret_cast<unsigned long long*>(group_q_len + kMaxRanked);  // one bit per vnode
  int* found = reinterpret_cast<int*>(joined + kMaxRanked / 64);
  const int tid = threadIdx.x;
  if (tid < n) views[tid] = load_vnode<GATHERED>(a, a.vnode_begin + tid);  // the block's own vnode is among them
  if (tid == 0) *found = -1;
  __syncthreads();
  // bit u: vnode u continues vnode u - 1 (same run, adjoining scratch rows).  Nothing is joined
  // while there are no more blocks than compute units: two half-filled blocks side by side
  // finish sooner than one full block.
  bool joins = false;
  if (tid > 0 && tid < n && 2LL * n * a.hkv * a.wide_chunks > a.block_slots) {
    const VnodeView& p = views[tid - 1];
    const VnodeView& c = views[tid];
    joins = p.kv_base == c.kv_base && p.kv_len == c.kv_len && p.q_off + p.q_len == c.q_off;
  }
  const unsigned long long wave_bits = __ballot(joins);
  if ((tid & 63) == 0) joined[tid >> 6] = wave_bits;
  __syncthreads();
  unsigned mine = 0;
  if (tid < n) {
    // first and last vnode of the chain of joined vnodes that holds this one
    int first = tid;
    for (int w = tid >> 6, hi = tid & 63; w >= 0; --w, hi = 63) {
      const unsigned long long stops = ~joined[w] & (hi == 63 ? ~0ull : ((2ull << hi) - 1));
      if (stops) {
        first = 64 * w + 63 - __builtin_clzll(stops);
        break;
      }
    }
    int last = n - 1;
    for (int u = tid + 1, w = u >> 6; w < (n + 63) / 64; ++w, u = 64 * w) {
      const unsigned long long stops = ~joined[w] & (~0ull << (u & 63));
      if (stops) {
        last = min(n, 64 * w + __builtin_ctzll(stops)) - 1;
        break;
      }
    }
    // groups of m vnodes from the start of the chain; the chain's first vnode is a full query tile
    const long long cap = (long long)kWideRows * a.wide_chunks;
    const long long tile_rows = max(1LL, (long long)views[first].q_len * a.g);
    const int m = (int)max(1LL, cap / tile_rows);
    const int head = first + (tid - first) / m * m;
    int q_len = 0;
    if (head == tid) {
      const VnodeView& tail = views[min(last, head + m - 1)];
      q_len = tail.q_off + tail.q_len - views[tid].q_off;
      const float work = (float)q_len * (float)a.g * (float)views[tid].kv_len;
      // (256 - tid is never 0: the key of a vnode without work must not be the 0 of "no group")
      static_assert(kMaxRanked <= 256, "the low nine bits of a key hold 256 - tid");
      mine = ((__builtin_bit_cast(unsigned, work) >> 8) << 9) | (unsigned)(256 - tid);
    }
    group_q_len[tid] = q_len;
  }
  keys[tid] = mine;  // all kMaxRanked entries: the vector reads below run over the padding
  __syncthreads();
  if (mine != 0) {
    int rank = 0;
    for (int j0 = 0; j0 < n; j0 += 16) {  // (keys past n are 0 and count for nothing)
      u32x4 k[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) k[i] = *reinterpret_cast<const u32x4*>(keys + j0 + 4 * i);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) rank += k[i][e] > mine ? 1 : 0;
    }
    if (rank == target) *found = tid;
  }
  __syncthreads();
  const int v = *found;
  if (v < 0) {  // more ranks than groups: an empty item
    view = VnodeView{0, 0, 0, 0};
    __syncthreads();
    return 0;
  }
  view = views[v];
  view.q_len = group_q_len[v];
  __syncthreads();  // the ranking area is reused as the staging ring
  return v;
}

// Launch order of the fused kernel.  Wide blocks come rank-major, then row chunk, kv head fastest
// (blocks that stream the same KV run are launched together and share it in L2); the narrow
// blocks follow and fill the machine while the wide blocks drain.
template <typename E, int D, bool GATHERED>
__global__ void __launch_bounds__(kWideBlock, D > 128 ? 1 : 512 / kWideBlock) stage1_fused_kernel(Stage1Args a) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int wide_blocks = a.prog_table ? a.num_programs * a.hkv : a.vnode_count * a.wide_chunks * a.hkv;
  const int wide_index = blockIdx.x, narrow_index = (int)blockIdx.x - wide_blocks;
  const bool is_wide = (int)blockIdx.x < wide_blocks;
  if (is_wide && a.prog_table) {
    // A block program written by the host, for one kv head (kv head fastest: the eight blocks of
    // a program land on the eight XCDs, and a head's K/V only ever enters one XCD's L2): its wide
    // vnodes one after the other, and its narrow vnodes, one wave each, before or after them.
    // Of the two blocks that share a compute unit one starts with its narrow vnodes and the
    // other ends with them, so that the memory-bound narrow vnodes of one run under the
    // arithmetic-bound wide vnodes of the other.
    const int program = wide_index / a.hkv;
    const int kvh = wide_index - program * a.hkv;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wide_first = a.prog_table[4 * program], wide_end = a.prog_table[4 * program + 1];
    const int narrow_first = a.prog_table[4 * program + 2], narrow_signed = a.prog_table[4 * program + 3];
    const int narrow_count = narrow_signed < 0 ? -narrow_signed : narrow_signed;
    auto narrow_vnodes = [&]() {
      for (int i = wave; i < narrow_count; i += kWideWaves)
        narrow_item<E, D, GATHERED>(a, smem, wave, 1, true, a.narrow_begin + narrow_first + i, kvh);
      __syncthreads();  // the waves' tiles become the ring of the next wide vnode
    };
    // the program's record, requested together with its table entry
    int* record = reinterpret_cast<int*>(smem + WideGeom<D>::kRecord);
    const bool with_records = !GATHERED && D <= 128 && a.prog_records != nullptr;   // launch uniform
    if (with_records) {
      record[threadIdx.x] = a.prog_records[(int64_t)program * kProgRecord + threadIdx.x];
      __syncthreads();
    }
    if (narrow_signed < 0) narrow_vnodes();
    for (int v = wide_first; v < wide_end; ++v) {
      if (with_records && narrow_signed >= 0 && v == wide_first && record[4] != 0) {
        const VnodeView vn{record[2], record[3], record[1], (int64_t)record[0]};
        wide_block<E, D, GATHERED>(a, smem, vn, kvh, 0, 1, record);
      } else {
        const VnodeView vn = load_vnode<GATHERED>(a, a.vnode_begin + v);
        wide_block<E, D, GATHERED>(a, smem, vn, kvh, 0, 1);
      }
    }
    if (narrow_signed > 0) narrow_vnodes();
  } else if (is_wide) {
    const int per_rank = a.wide_chunks * a.hkv;
    const int rank = wide_index / per_rank;
    const int rest = wide_index - rank * per_rank;
    // Launch slot `rest / hkv` of a rank serves chunk (slot + rank / 2) % chunks.  Consecutive
    // blocks of one kv head go round robin to the four shader engines of an XCD, strictly in
    // order (a block waits for its engine even when others have room); without the rotation an
    // engine would only ever get first chunks, which run longer than last ones.
    const int slot = rest / a.hkv;
    const int chunk = (slot + (rank >> 1)) % a.wide_chunks;
    VnodeView vn;
    (void)wide_vnode_of_rank<GATHERED>(a, smem, rank, vn);
    wide_block<E, D, GATHERED>(a, smem, vn, rest - slot * a.hkv, chunk, a.wide_chunks);
  } else {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int share = a.narrow_share;
    const int item = narrow_index * (kWideWaves / share) + wave / share + a.narrow_in_programs * a.hkv;
    const bool exists = item < a.narrow_count * a.hkv;
    if (share == 1 && !exists) return;  // whole wave; no block barrier below in this mode
    const int local_vnode = item / a.hkv;
    const int kvh = item - local_vnode * a.hkv;
    narrow_item<E, D, GATHERED>(a, smem, wave, share, exists, a.narrow_begin + local_vnode, kvh);
  }
}

// ---------------------------------------------------------------------------------------
// DeFT-Flatten's first stage (the comparison engine of the reference's benchmark,
// kernel_bench/DeFT.py:194-340): one block per (subtree, kv head).  A subtree is a run of
// consecutive tokens of the depth-first token order (128 in the benchmark) that may span
// several tree nodes; its query set holds every request that attends any of its tokens, and a
// 64-bit word per (group of mask_len requests, token) says which requests of the group attend the
// token.  The block keeps up to 128 tokens of the subtree in LDS (the two super-tile buffers of
// the wide kernel, same layout, same direct loads) and passes its query rows over them 128 at a
// time, 32 per wave, with the scores of tokens a row does not attend set to a large negative
// value before the soft-max (DeFT.py:283-306).  The partial output is rounded to fp16 on its
// way to the fp32 scratch, as the reference kernel does (DeFT.py:391).
// ---------------------------------------------------------------------------------------
struct DeftArgs {
  Stage1Args s;                    // tensors, strides, the six vnode lists (vnode = subtree), scale, scratch
  const int64_t* causalmask;       // per subtree: [groups of mask_len requests][kv_len] words
  const int32_t* causalmask_offset;
  int mask_len;                    // requests per mask word: a power of two, at most 64
  int num_subtrees;
};

constexpr int kDeftChunk = 2 * 64;       // tokens held in LDS at a time (both ring buffers)
// Raw score of a token a row does not attend (the reference writes -1e6 over the scaled score,
// DeFT.py:306).  Finite and moderate on purpose: a tile in which a row attends nothing makes this
// value the row's soft-max reference, and the probabilities of that tile come out as exp2 of the
// rounding error of (score * scale) -- about 1 for this magnitude, infinite for a huge one.  They
// are garbage either way and are wiped out (factor exp2(-1e5) = 0) by the first attended token.
constexpr float kDeftMasked = -1.0e6f;
constexpr int kDeftMaskGroups = 5;       // mask groups 128 consecutive query rows can touch (g = 1, mask_len 32: 4 + 1)

template <typename E, int D>
__global__ void __launch_bounds__(kWideBlock, D > 128 ? 1 : 2) deft_stage1_kernel(DeftArgs d) {
  using W = WideGeom<D>;
  const Stage1Args& a = d.s;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int subtree = blockIdx.x / a.hkv;
  const int kvh = blockIdx.x - subtree * a.hkv;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const VnodeView vn = load_vnode<false>(a, subtree);
  const int rows_total = vn.q_len * a.g;
  const int64_t* masks = d.causalmask + d.causalmask_offset[subtree];
  const int grp_row = lane / W::kChunks, pos = lane % W::kChunks;
  const char* kbase = a.k + 2 * ((int64_t)kvh * a.sk1);
  const char* vbase = a.v + 2 * ((int64_t)kvh * a.sv1);
  const unsigned k_stride = (unsigned)(2 * a.sk0), v_stride = (unsigned)(2 * a.sv0);
  const unsigned ring = lds_offset(smem);
  // the mask words of the chunk in LDS, after the ring: [kDeftMaskGroups][kDeftChunk] 64-bit words
  uint32_t* mask_lds = reinterpret_cast<uint32_t*>(smem + W::kRing);
  const unsigned mask_lds_addr = ring + W::kRing;
  WideLane la0;
  init_lane<D>(la0, ring);
  const int nchunks = (vn.kv_len + kDeftChunk - 1) / kDeftChunk;
  const int h = lane >> 5;

  for (int row0 = 0; row0 < rows_total; row0 += kWideRows) {
    const int my_row0 = row0 + 32 * wave;
    const bool active = my_row0 < rows_total;
    const char* q_src = q_row_address32<false>(a, vn, kvh, active ? my_row0 : rows_total);
    u32x4 qf[D / 16];
    load_q_frags32<D>(q_src, qf);
    WideState<D> st;
    reset_state<D>(st);
    // the lane's request within the subtree's query set, its mask group and its bit in the group's words
    const int my_req = min(my_row0 + (lane & 31), rows_total - 1) / a.g;
    const int first_group = (row0 / a.g) / d.mask_len;
    const int groups_here = min((min(row0 + kWideRows, rows_total) - 1) / a.g / d.mask_len - first_group + 1, kDeftMaskGroups);
    const int my_group = min(my_req / d.mask_len - first_group, kDeftMaskGroups - 1);
    const int my_bit = my_req & (d.mask_len - 1);
    const bool upper = my_bit >= 32;
    const unsigned bit = 1u << (my_bit & 31);
    for (int chunk = 0; chunk < nchunks; ++chunk) {
      const int c0 = chunk * kDeftChunk;
      const int here = min(kDeftChunk, vn.kv_len - c0);
      __syncthreads();   // the previous pass (or chunk) is out of LDS
      if (row0 == 0 || nchunks > 1) {
        // K and V rows of the chunk: 2 x 16 groups of 1 KB per super tile, dealt to the four waves
        // (tokens past the end repeat the last one: their scores are masked)
#pragma unroll
        for (int sup = 0; sup < 2; ++sup)
#pragma unroll
          for (int u = 0; u < W::kUnits; ++u) {
            const bool is_v = W::kGroups >= kWideWaves ? u >= W::kSlots : wave >= W::kGroups;
            const int sl = u % W::kSlots;
            const int grp = W::kGroups >= kWideWaves ? sl * kWideWaves + wave : wave % W::kGroups;
            const int row = grp * W::kGroupRows + grp_row;
            const int t = min(c0 + sup * W::kTokens + row, vn.kv_len - 1);
            const unsigned slot = (unsigned)a.kv_entries[vn.kv_base + t];
            const char* src = (is_v ? vbase : kbase) + (uint64_t)slot * (is_v ? v_stride : k_stride);
            load_direct16(src + 16 * (pos ^ W::swz(row)), ring + sup * W::kBytes + (is_v ? W::kBytesK : 0) + grp * 1024);
          }
      }
      // the mask words of this pass's groups for the chunk's tokens (zero past the subtree)
      for (int i = threadIdx.x; i < groups_here * kDeftChunk; i += kWideBlock) {
        const int gsel = i / kDeftChunk, t = i - gsel * kDeftChunk;
        const int64_t word = t < here ? masks[(int64_t)(first_group + gsel) * vn.kv_len + c0 + t] : 0;
        mask_lds[2 * i] = (uint32_t)(uint64_t)word;
        mask_lds[2 * i + 1] = (uint32_t)((uint64_t)word >> 32);
      }
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): rows landed (and the Q fragments)
      __syncthreads();
      if (active) {
        const int tiles = (here + kTileTokens - 1) / kTileTokens;
        for (int tile = 0; tile < tiles; ++tile) {
          // the lane's 16 tokens of the tile are four runs of four consecutive ones: 32 bytes of mask words each
          const unsigned words = mask_lds_addr + 8u * (unsigned)(my_group * kDeftChunk + tile * kTileTokens + 4 * h);
          auto mask = [&](f32x16& sc) {
#pragma unroll
            for (int quad = 0; quad < 4; ++quad) {
              const u32x4 w0 = lds_read16(words + 64u * quad), w1 = lds_read16(words + 64u * quad + 16u);
              const unsigned m4[4] = {upper ? w0[1] : w0[0], upper ? w0[3] : w0[2], upper ? w1[1] : w1[0], upper ? w1[3] : w1[2]};
#pragma unroll
              for (int jj = 0; jj < 4; ++jj) sc[4 * quad + jj] = (m4[jj] & bit) ? sc[4 * quad + jj] : kDeftMasked;
            }
          };
          const WideLane la = at_buffer(la0, (unsigned)(tile >> 1) * W::kBytes);
          tile_step32<E, D>(la, (tile & 1) * W::kTileBytes, here - tile * kTileTokens, a.scale_log2, qf, st, mask);
        }
      }
    }
    finish_state<D>(st);
    // (the reference rounds the normalised partial output to fp16 before it stores it, DeFT.py:391)
    if (active) write_partials32<D, true>(a, vn, kvh, my_row0, st);
  }
}

// ---------------------------------------------------------------------------------------
// Stage 2
// ---------------------------------------------------------------------------------------
struct Stage2Args {
  const int32_t* req_entries;
  const int32_t* req_offs;
  const int32_t* req_lens;
  const float* mid_o;
  int64_t so0, so1;
  const float* mid_lse;
  int64_t sl0;
  char* o;
  int64_t oo0, oo1;
  int batch, hq;
  int nsplit;  // > 0: gathered mode, request r owns rows [r*nsplit, (r+1)*nsplit)
  // (or null) one record of kReqRecord int32 per request, written by the host: req_lens[r],
  // req_offs[r], then the request's first kReqRecord - 2 entries -- what the block needs before
  // it can ask for the partial rows, in one memory round trip instead of two
  const int32_t* req_table;
};
constexpr int kReqRecord = 16;
constexpr int kReqRecEntries = kReqRecord - 2;

template <int WIDTH> __device__ __forceinline__ float group_max(float x) {
#pragma unroll
  for (int d = WIDTH / 2; d >= 1; d >>= 1) x = fmaxf(x, __shfl_xor(x, d, WIDTH));
  return x;
}
template <int WIDTH> __device__ __forceinline__ float group_sum(float x) {
#pragma unroll
  for (int d = WIDTH / 2; d >= 1; d >>= 1) x += __shfl_xor(x, d, WIDTH);
  return x;
}

// A group of D/4 lanes owns one (request, head): lane i fetches the row index and the
// log-sum-exp of partial i, the group reduces max and weight sum with shuffles, then every
// lane accumulates its own 4 output dims over the partials, taking weight and row index of
// partial i from lane i.
template <typename E, int D>
__global__ void __launch_bounds__(kBlock) stage2_kernel(Stage2Args a) {
  constexpr int LPH = D / 4;
  constexpr int HPB = kBlock / LPH;
  const int grp = threadIdx.x / LPH, gl = threadIdx.x % LPH;
  const int req = blockIdx.x;
  const int head = blockIdx.y * HPB + grp;
  if (head >= a.hq) return;
  const int32_t* rec = a.req_table ? a.req_table + (int64_t)req * kReqRecord : nullptr;  // launch uniform
  int off, n, rec_row = -1;
  if (a.nsplit > 0) {
    off = req * a.nsplit;
    n = a.nsplit;
  } else if (rec) {
    n = rec[0];
    off = rec[1];
    rec_row = rec[2 + min(gl, kReqRecEntries - 1)];  // (requested together with the two words above)
  } else {
    off = a.req_offs[req];
    n = a.req_lens[req];
  }

  float m_run = -INFINITY, l_run = 0.f;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int base = 0; base < n; base += LPH) {
    const int cnt = min(LPH, n - base);
    int my_row = -1;
    if (gl < cnt) {
      if (a.nsplit > 0) my_row = off + base + gl;
      else if (rec && base + gl < kReqRecEntries) my_row = base == 0 ? rec_row : rec[2 + base + gl];
      else my_row = a.req_entries[off + base + gl];
    }
    // Rows in batches of kBatch, all loads of a batch issued before the first is used (the rows
    // are in bounds whatever their weight; a zero weight discards the row's contents).  The
    // first batch is requested together with the log-sum-exp values, not after them: both
    // depend on the row indices only.
    constexpr int kBatch = 8;
    f32x4 part[kBatch];
    auto request = [&](int i0) {
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const int ri = __shfl(my_row, min(i0 + j, cnt - 1), LPH);
        part[j] = *reinterpret_cast<const f32x4*>(a.mid_o + (int64_t)ri * a.so0 + (int64_t)head * a.so1 + 4 * gl);
      }
    };
    float my_lse = -INFINITY;
    if (gl < cnt) my_lse = a.mid_lse[(int64_t)my_row * a.sl0 + head];
    request(0);
    const float m_new = fmaxf(m_run, group_max<LPH>(my_lse));
    const float w = (my_lse == -INFINITY) ? 0.f : __expf(my_lse - m_new);
    const float keep = (m_run == -INFINITY) ? 0.f : __expf(m_run - m_new);
    l_run = l_run * keep + group_sum<LPH>(w);
    acc *= keep;
    m_run = m_new;
    for (int i0 = 0; i0 < cnt; i0 += kBatch) {
      if (i0 > 0) request(i0);
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const float wi = (i0 + j < cnt) ? __shfl(w, min(i0 + j, cnt - 1), LPH) : 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += (wi != 0.f) ? part[j][e] * wi : 0.f;
      }
    }
  }
  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
  acc *= inv;
  u32x2 out = {E::pack2(acc[0], acc[1]), E::pack2(acc[2], acc[3])};
  *reinterpret_cast<u32x2*>(a.o + 2 * ((int64_t)req * a.oo0 + (int64_t)head * a.oo1 + 4 * gl)) = out;
}

// ---------------------------------------------------------------------------------------
// The step's new K and V rows into the pools (one launch for both)
// ---------------------------------------------------------------------------------------
struct StoreArgs {
  const char* k_new;
  const char* v_new;
  int64_t kn0, kn1, vn0, vn1;  // element strides of the new rows [tokens, Hkv, D]
  const void* loc;             // pool slot per token, int32 or int64
  int loc_is_int64;
  char* k_pool;
  char* v_pool;
  int64_t sk0, sk1, sv0, sv1;
  int64_t num_slots;
  int tokens, hkv, chunks;     // chunks = 16-byte pieces per (token, head) row
};

// One thread moves 16 bytes of a K row and the same 16 bytes of the V row.  A token whose slot
// lies outside the pool is skipped.
__global__ void __launch_bounds__(256) store_kv_kernel(StoreArgs a) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int per_token = a.hkv * a.chunks;
  const int64_t token = i / per_token;
  if (token >= a.tokens) return;
  const int rest = (int)(i - token * per_token);
  const int head = rest / a.chunks, chunk = rest - head * a.chunks;
  const int64_t slot = a.loc_is_int64 ? static_cast<const int64_t*>(a.loc)[token]
                                      : (int64_t) static_cast<const int32_t*>(a.loc)[token];
  if (slot < 0 || slot >= a.num_slots) return;
  const u32x4 kx = *reinterpret_cast<const u32x4*>(a.k_new + 2 * (token * a.kn0 + head * a.kn1) + 16 * chunk);
  const u32x4 vx = *reinterpret_cast<const u32x4*>(a.v_new + 2 * (token * a.vn0 + head * a.vn1) + 16 * chunk);
  *reinterpret_cast<u32x4*>(a.k_pool + 2 * (slot * a.sk0 + head * a.sk1) + 16 * chunk) = kx;
  *reinterpret_cast<u32x4*>(a.v_pool + 2 * (slot * a.sv0 + head * a.sv1) + 16 * chunk) = vx;
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------
constexpr int kMaxDevices = 64;
inline int current_device() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) (void)hipGetLastError();
  return dev >= 0 && dev < kMaxDevices ? dev : 0;
}
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename E, int D, int NQB, bool SPLIT, bool GATHERED>
int launch_stage1_inst(const Stage1Args& a, int hkv, hipStream_t stream) {
  const size_t lds = (size_t)kWavesPerBlock * TileGeom<D>::kBytes;
  auto kern = stage1_kernel<E, D, NQB, SPLIT, GATHERED>;
  // (raising the dynamic LDS limit is idempotent: two threads that both find the flag clear both raise it)
  static std::atomic<bool> configured_on[kMaxDevices];
  std::atomic<bool>& configured = configured_on[current_device()];
  if (!configured.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
      (void)hipGetLastError();
      return FT_ERR_LAUNCH;
    }
    configured.store(true, std::memory_order_release);
  }
  const unsigned gx = SPLIT ? (unsigned)a.vnode_count : (unsigned)((a.vnode_count + kWavesPerBlock - 1) / kWavesPerBlock);
  hipLaunchKernelGGL(kern, dim3(gx, (unsigned)hkv, 1), dim3(kBlock, 1, 1), lds, stream, a);
  return hipGetLastError() == hipSuccess ? FT_OK : FT_ERR_LAUNCH;
}

// Waves that share one narrow vnode: the largest power of two (at most a block's four) that
// fills at most three quarters of the wave slots (8 per compute unit).  With far fewer vnodes than slots the
// waves would each walk a long run alone, one memory round trip per tile; with the slots nearly
// full the runs are limited by memory bandwidth already and sharing only adds barriers.
inline int wave_slots() {
  // per device; threads that race on the first call compute and store the same value
  static std::atomic<int> slots_on[kMaxDevices];
  std::atomic<int>& slots = slots_on[current_device()];
  int n = slots.load(std::memory_order_relaxed);
  if (n == 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
      (void)hipGetLastError();
      cus = 256;
    }
    n = cus * kWaveSlotsPerCu;
    slots.store(n, std::memory_order_relaxed);
  }
  return n;
}
inline int narrow_share_for(int64_t items, int head_dim) {
  const int slots = head_dim > 128 ? wave_slots() / 2 : wave_slots();   // (one block per compute unit at 512-byte rows)
  int share = 1;
  while (share < kWideWaves && 4 * items * (2 * share) <= 3 * (int64_t)slots) share *= 2;
  return share;
}

template <typename E, int D, bool GATHERED>
int launch_stage1_fused(const Stage1Args& a0, hipStream_t stream) {
  constexpr size_t kWideLds = (size_t)WideGeom<D>::kLds;
  constexpr size_t kNarrowLds = (size_t)kWideWaves * NarrowGeom<D>::kLds;
  constexpr size_t lds = kWideLds > kNarrowLds ? kWideLds : kNarrowLds;
  auto kern = stage1_fused_kernel<E, D, GATHERED>;
  // (raising the dynamic LDS limit is idempotent: two threads that both find the flag clear both raise it)
  static std::atomic<bool> configured_on[kMaxDevices];
  std::atomic<bool>& configured = configured_on[current_device()];
  if (!configured.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
      (void)hipGetLastError();
      return FT_ERR_LAUNCH;
    }
    configured.store(true, std::memory_order_release);
  }
  Stage1Args a = a0;
  const int64_t narrow_items = (int64_t)(a.narrow_count - a.narrow_in_programs) * a.hkv;  // those of the trailing blocks
  a.narrow_share = narrow_share_for(narrow_items, D);
  const int per_block = kWideWaves / a.narrow_share;
  const int64_t narrow_blocks = (narrow_items + per_block - 1) / per_block;
  a.wide_chunks = std::max(1, std::min(8, (a.wide_rows + kWideRows - 1) / kWideRows));
  a.block_slots = (D > 128 ? wave_slots() / 2 : wave_slots()) / kWideWaves;
  const int64_t wide_blocks = a.prog_table ? (int64_t)a.num_programs * a.hkv : (int64_t)a.vnode_count * a.wide_chunks * a.hkv;
  const int64_t blocks = wide_blocks + narrow_blocks;
  if (blocks == 0) return FT_OK;
  if (blocks > INT32_MAX) return FT_ERR_ARGUMENT;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks, 1, 1), dim3(kWideBlock, 1, 1), lds, stream, a);
  return hipGetLastError() == hipSuccess ? FT_OK : FT_ERR_LAUNCH;
}

template <typename E, int D, bool GATHERED>
int launch_stage1_narrow(const Stage1Args& a0, hipStream_t stream) {
  Stage1Args a = a0;
  const int64_t blocks = (int64_t)a.narrow_count * a.hkv;
  if (blocks == 0) return FT_OK;
  if (blocks > INT32_MAX) return FT_ERR_ARGUMENT;
  a.narrow_share = narrow_share_for(blocks, D);
  auto kern = stage1_narrow_kernel<E, D, GATHERED>;
  const size_t lds = (size_t)a.narrow_share * NarrowGeom<D>::kLds;
  // (raising the dynamic LDS limit is idempotent: two threads that both find the flag clear both raise it)
  static std::atomic<bool> configured_on[kMaxDevices];
  std::atomic<bool>& configured = configured_on[current_device()];
  if (!configured.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            kWideWaves * NarrowGeom<D>::kLds) != hipSuccess) {
      (void)hipGetLastError();
      return FT_ERR_LAUNCH;
    }
    configured.store(true, std::memory_order_release);
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks, 1, 1), dim3(kWave * a.narrow_share, 1, 1), lds, stream, a);
  return hipGetLastError() == hipSuccess ? FT_OK : FT_ERR_LAUNCH;
}

// `a` names two vnode ranges: [vnode_begin, +vnode_count) of wide vnodes (more than 16 query
// rows) and [narrow_begin, +narrow_count) of narrow ones.
template <typename E, int D, bool GATHERED, bool STAGED = false>
int launch_stage1_d(const Stage1Args& a, hipStream_t stream) {
  if constexpr (STAGED) {
    // 128-token double buffers of 512-byte rows do not fit in LDS: per-wave staging kernels
    if (a.vnode_count > 0)
      if (int rc = launch_stage1_inst<E, D, 2, true, GATHERED>(a, a.hkv, stream)) return rc;
    if (a.narrow_count > 0) {
      Stage1Args n = a;
      n.vnode_begin = a.narrow_begin;
      n.vnode_count = a.narrow_count;
      return launch_stage1_inst<E, D, 1, false, GATHERED>(n, a.hkv, stream);
    }
    return FT_OK;
  } else {
    if (a.vnode_count == 0 && !a.prog_table) return launch_stage1_narrow<E, D, GATHERED>(a, stream);
    return launch_stage1_fused<E, D, GATHERED>(a, stream);
  }
}

template <bool GATHERED>
int launch_stage1(const Stage1Args& a, int d, int dtype, hipStream_t stream) {
#define FT_DISPATCH_D(E)                                              \
  switch (d) {                                                        \
    case 16: return launch_stage1_d<E, 32, GATHERED, true>(a, stream);\
    case 32: return launch_stage1_d<E, 32, GATHERED>(a, stream);      \
    case 64: return launch_stage1_d<E, 64, GATHERED>(a, stream);      \
    case 128: return launch_stage1_d<E, 128, GATHERED>(a, stream);    \
    case 256: return launch_stage1_d<E, 256, GATHERED>(a, stream);    \
    default: return FT_ERR_HEAD_DIM;                                  \
  }
  if (dtype == FT_DTYPE_F16) { FT_DISPATCH_D(F16) }
  if (dtype == FT_DTYPE_BF16) { FT_DISPATCH_D(BF16) }
#undef FT_DISPATCH_D
  return FT_ERR_DTYPE;
}

template <typename E, int D>
int launch_stage2_inst(const Stage2Args& a, hipStream_t stream) {
  constexpr int HPB = kBlock / (D / 4);
  hipLaunchKernelGGL((stage2_kernel<E, D>), dim3((unsigned)a.batch, (unsigned)((a.hq + HPB - 1) / HPB), 1),
                     dim3(kBlock, 1, 1), 0, stream, a);
  return hipGetLastError() == hipSuccess ? FT_OK : FT_ERR_LAUNCH;
}

int launch_stage2(const Stage2Args& a, int d, int dtype, hipStream_t stream) {
#define FT_DISPATCH_D(E)                                       \
  switch (d) {                                                 \
    case 16: return launch_stage2_inst<E, 16>(a, stream);      \
    case 32: return launch_stage2_inst<E, 32>(a, stream);      \
    case 64: return launch_stage2_inst<E, 64>(a, stream);      \
    case 128: return launch_stage2_inst<E, 128>(a, stream);    \
    case 256: return launch_stage2_inst<E, 256>(a, stream);    \
    default: return FT_ERR_HEAD_DIM;                           \
  }
  if (dtype == FT_DTYPE_F16) { FT_DISPATCH_D(F16) }
  if (dtype == FT_DTYPE_BF16) { FT_DISPATCH_D(BF16) }
#undef FT_DISPATCH_D
  return FT_ERR_DTYPE;
}

template <typename E, int D>
int launch_deft_inst(const DeftArgs& d, hipStream_t stream) {
  constexpr size_t lds = (size_t)WideGeom<D>::kLds;
  static_assert(kDeftMaskGroups * kDeftChunk * 8 <= 4 * WideGeom<D>::kIdxCap, "the mask words share the index area");
  auto kern = deft_stage1_kernel<E, D>;
  static std::atomic<bool> configured_on[kMaxDevices];
  std::atomic<bool>& configured = configured_on[current_device()];
  if (!configured.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
      (void)hipGetLastError();
      return FT_ERR_LAUNCH;
    }
    configured.store(true, std::memory_order_release);
  }
  const int64_t blocks = (int64_t)d.num_subtrees * d.s.hkv;
  if (blocks == 0) return FT_OK;
  if (blocks > INT32_MAX) return FT_ERR_ARGUMENT;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks, 1, 1), dim3(kWideBlock, 1, 1), lds, stream, d);
  return hipGetLastError() == hipSuccess ? FT_OK : FT_ERR_LAUNCH;
}

int launch_deft(const DeftArgs& d, int head_dim, int dtype, hipStream_t stream) {
#define FT_DISPATCH_D(E)                                         \
  switch (head_dim) {                                            \
    case 32: return launch_deft_inst<E, 32>(d, stream);          \
    case 64: return launch_deft_inst<E, 64>(d, stream);          \
    case 128: return launch_deft_inst<E, 128>(d, stream);        \
    case 256: return launch_deft_inst<E, 256>(d, stream);        \
    default: return FT_ERR_HEAD_DIM;                             \
  }
  if (dtype == FT_DTYPE_F16) { FT_DISPATCH_D(F16) }
  if (dtype == FT_DTYPE_BF16) { FT_DISPATCH_D(BF16) }
#undef FT_DISPATCH_D
  return FT_ERR_DTYPE;
}

int check_common(int d, int g, int dtype) {
  if (dtype != FT_DTYPE_F16 && dtype != FT_DTYPE_BF16) return FT_ERR_DTYPE;
  if (d != 16 && d != 32 && d != 64 && d != 128 && d != 256) return FT_ERR_HEAD_DIM;
  if (g < 1 || g > 64) return FT_ERR_GROUP;
  return FT_OK;
}

}  // namespace

// ---------------------------------------------------------------------------------------
// Scratch of ft_decode_static: the partial results of one decode call (mid_o, then mid_lse) in
// a device array of the library, for callers that cannot allocate.  Every device the library
// runs on holds its own copy until the process ends.  In host code the array's name is a
// stand-in, not a device address: the address on the current device is asked for once per
// device and kept, and only that pointer is handed to kernels.
// ---------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[FT_STATIC_SCRATCH_BYTES];

static int static_scratch_of_current_device(char** out) {
  constexpr int kMaxDevices = 64;
  // No lock: the lookup gives every thread the same address for a device, so threads that race on
  // a device's first call store the same pointer, and later calls are one atomic load.
  static std::atomic<char*> address[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return FT_ERR_LAUNCH;
  }
  char* ptr = address[dev].load(std::memory_order_acquire);
  if (!ptr) {
    if (hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
      (void)hipGetLastError();
      return FT_ERR_LAUNCH;
    }
    address[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return FT_OK;
}

extern "C" {

const char* ft_version(void) { return "fasttree_hip 0.1 (gfx950)"; }

int64_t ft_static_scratch_bytes(void) { return (int64_t)FT_STATIC_SCRATCH_BYTES; }

const char* ft_error_string(int code) {
  switch (code) {
    case FT_OK: return "ok";
    case FT_ERR_NULL_POINTER: return "null pointer argument";
    case FT_ERR_DTYPE: return "unsupported dtype (fp16 and bf16 only)";
    case FT_ERR_HEAD_DIM: return "unsupported head dimension (16, 32, 64, 128, 256)";
    case FT_ERR_GROUP: return "unsupported query/KV head ratio";
    case FT_ERR_ALIGNMENT: return "pointer or stride not aligned as required";
    case FT_ERR_ARGUMENT: return "argument out of range";
    case FT_ERR_LAUNCH: return "kernel launch failed";
    case FT_ERR_SCRATCH: return "partial results do not fit the library's static scratch (FT_STATIC_SCRATCH_BYTES)";
    default: return "unknown error";
  }
}

// Validates the stage-1 arguments shared by ft_stage1 and ft_decode and fills everything of
// `a` but the vnode ranges.
static int stage1_setup(Stage1Args& a, const void* q, const void* k, const void* v,
                        int64_t sq0, int64_t sq1, int64_t sk0, int64_t sk1, int64_t sv0, int64_t sv1,
                        const int32_t* vnode_to_kv_entries, const int32_t* vnode_to_kv_offs,
                        const int32_t* vnode_to_kv_lens, const int32_t* vnode_to_q_entries,
                        const int32_t* vnode_to_q_offs, const int32_t* vnode_to_q_lens,
                        int num_kv_heads, int kv_group_num, int head_dim, float sm_scale,
                        float* mid_o, int64_t so0, int64_t so1, float* mid_lse, int64_t sl0, int dtype) {
  if (int rc = check_common(head_dim, kv_group_num, dtype)) return rc;
  if (!q || !k || !v || !vnode_to_kv_entries || !vnode_to_kv_offs || !vnode_to_kv_lens || !vnode_to_q_entries ||
      !vnode_to_q_offs || !vnode_to_q_lens || !mid_o || !mid_lse)
    return FT_ERR_NULL_POINTER;
  if (num_kv_heads < 1 || num_kv_heads > 65535 || !(sm_scale > 0.f)) return FT_ERR_ARGUMENT;
  // the kernels form row addresses as slot * (32-bit byte stride)
  if (sk0 < 0 || sv0 < 0 || sk0 >= (int64_t(1) << 31) || sv0 >= (int64_t(1) << 31)) return FT_ERR_ARGUMENT;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(mid_o) || (sq0 | sq1 | sk0 | sk1 | sv0 | sv1) % 8 != 0 ||
      (so0 | so1) % 4 != 0)
    return FT_ERR_ALIGNMENT;
  a = Stage1Args{};
  a.q = static_cast<const char*>(q);
  a.k = static_cast<const char*>(k);
  a.v = static_cast<const char*>(v);
  a.sq0 = sq0; a.sq1 = sq1; a.sk0 = sk0; a.sk1 = sk1; a.sv0 = sv0; a.sv1 = sv1;
  a.kv_entries = vnode_to_kv_entries; a.kv_offs = vnode_to_kv_offs; a.kv_lens = vnode_to_kv_lens;
  a.q_entries = vnode_to_q_entries; a.q_offs = vnode_to_q_offs; a.q_lens = vnode_to_q_lens;
  a.g = kv_group_num;
  a.hkv = num_kv_heads;
  a.real_dim = head_dim;
  a.scale_log2 = sm_scale * kLog2e;
  a.mid_o = mid_o; a.so0 = so0; a.so1 = so1; a.mid_lse = mid_lse; a.sl0 = sl0;
  return FT_OK;
}

// A phase whose tile holds at most 16 query rows is served one wave per (vnode, KV head).
static bool is_narrow(int q_tile, int kv_group_num) { return (int64_t)q_tile * kv_group_num <= 16; }

static bool range_ok(int begin, int count, int num_kv_heads) {
  return begin >= 0 && count >= 0 && (int64_t)count * num_kv_heads <= INT32_MAX;
}

int ft_stage1(const void* q, const void* k, const void* v,
              int64_t sq0, int64_t sq1, int64_t sk0, int64_t sk1, int64_t sv0, int64_t sv1,
              const int32_t* vnode_to_kv_entries, const int32_t* vnode_to_kv_offs,
              const int32_t* vnode_to_kv_lens, const int32_t* vnode_to_q_entries,
              const int32_t* vnode_to_q_offs, const int32_t* vnode_to_q_lens,
              int vnode_begin, int vnode_count, int num_kv_heads, int kv_group_num, int head_dim,
              int q_tile, int kv_tile, float sm_scale,
              float* mid_o, int64_t so0, int64_t so1, float* mid_lse, int64_t sl0,
              int dtype, ft_stream_t stream) {
  (void)kv_tile;
  if (int rc = check_common(head_dim, kv_group_num, dtype)) return rc;
  if (vnode_count == 0) return FT_OK;
  Stage1Args a;
  if (int rc = stage1_setup(a, q, k, v, sq0, sq1, sk0, sk1, sv0, sv1, vnode_to_kv_entries, vnode_to_kv_offs,
                            vnode_to_kv_lens, vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens, num_kv_heads,
                            kv_group_num, head_dim, sm_scale, mid_o, so0, so1, mid_lse, sl0, dtype))
    return rc;
  if (q_tile < 1 || !range_ok(vnode_begin, vnode_count, num_kv_heads)) return FT_ERR_ARGUMENT;
  if (is_narrow(q_tile, kv_group_num)) {
    a.narrow_begin = vnode_begin; a.narrow_count = vnode_count;
  } else {
    a.vnode_begin = vnode_begin; a.vnode_count = vnode_count;
    a.wide_rows = (int)std::min<int64_t>((int64_t)q_tile * kv_group_num, 1 << 20);
  }
  return launch_stage1<false>(a, head_dim, dtype, stream);
}

static int stage2_with_table(const int32_t* req_to_vnode_entries, const int32_t* req_to_vnode_offs,
                             const int32_t* req_to_vnode_lens, const int32_t* req_table,
                             const float* mid_o, int64_t so0, int64_t so1, const float* mid_lse, int64_t sl0,
                             void* o, int64_t oo0, int64_t oo1,
                             int batch_size, int num_qo_heads, int head_dim, int dtype, ft_stream_t stream) {
  if (int rc = check_common(head_dim, 1, dtype)) return rc;
  if (batch_size == 0) return FT_OK;
  if (!req_to_vnode_entries || !req_to_vnode_offs || !req_to_vnode_lens || !mid_o || !mid_lse || !o)
    return FT_ERR_NULL_POINTER;
  if (batch_size < 0 || num_qo_heads < 1) return FT_ERR_ARGUMENT;
  if (!aligned16(mid_o) || !aligned16(o) || (so0 | so1) % 4 != 0 || (oo0 | oo1) % 4 != 0) return FT_ERR_ALIGNMENT;
  Stage2Args a{};
  a.req_entries = req_to_vnode_entries; a.req_offs = req_to_vnode_offs; a.req_lens = req_to_vnode_lens;
  a.mid_o = mid_o; a.so0 = so0; a.so1 = so1; a.mid_lse = mid_lse; a.sl0 = sl0;
  a.o = static_cast<char*>(o); a.oo0 = oo0; a.oo1 = oo1;
  a.batch = batch_size; a.hq = num_qo_heads; a.nsplit = 0;
  a.req_table = req_table;
  return launch_stage2(a, head_dim, dtype, stream);
}

int ft_stage2(const int32_t* req_to_vnode_entries, const int32_t* req_to_vnode_offs,
              const int32_t* req_to_vnode_lens,
              const float* mid_o, int64_t so0, int64_t so1, const float* mid_lse, int64_t sl0,
              void* o, int64_t oo0, int64_t oo1,
              int batch_size, int num_qo_heads, int head_dim, int dtype, ft_stream_t stream) {
  return stage2_with_table(req_to_vnode_entries, req_to_vnode_offs, req_to_vnode_lens, nullptr, mid_o, so0, so1, mid_lse,
                           sl0, o, oo0, oo1, batch_size, num_qo_heads, head_dim, dtype, stream);
}

int ft_stage1_phases(const void* q, const void* k, const void* v,
                     int64_t sq0, int64_t sq1, int64_t sk0, int64_t sk1, int64_t sv0, int64_t sv1,
                     const int32_t* vnode_to_kv_entries, const int32_t* vnode_to_kv_offs,
                     const int32_t* vnode_to_kv_lens, const int32_t* vnode_to_q_entries,
                     const int32_t* vnode_to_q_offs, const int32_t* vnode_to_q_lens,
                     float* mid_o, int64_t so0, int64_t so1, float* mid_lse, int64_t sl0,
                     const int32_t phase_node_nums[2], const int32_t phase_node_offsets[2],
                     const int32_t phase_q_tile_sizes[2], const int32_t phase_kv_tile_sizes[2],
                     int num_qo_heads, int num_kv_heads, int head_dim,
                     float sm_scale, int dtype, ft_stream_t stream) {
  if (!phase_node_nums || !phase_node_offsets || !phase_q_tile_sizes || !phase_kv_tile_sizes) return FT_ERR_NULL_POINTER;
  if (num_kv_heads < 1 || num_qo_heads % num_kv_heads != 0) return FT_ERR_GROUP;
  const int g = num_qo_heads / num_kv_heads;
  if (int rc = check_common(head_dim, g, dtype)) return rc;
  if (phase_node_nums[0] == 0 && phase_node_nums[1] == 0) return FT_OK;
  Stage1Args a;
  if (int rc = stage1_setup(a, q, k, v, sq0, sq1, sk0, sk1, sv0, sv1, vnode_to_kv_entries, vnode_to_kv_offs,
                            vnode_to_kv_lens, vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens, num_kv_heads, g,
                            head_dim, sm_scale, mid_o, so0, so1, mid_lse, sl0, dtype))
    return rc;
  const bool pending[2] = {phase_node_nums[0] != 0, phase_node_nums[1] != 0};
  for (int phase = 0; phase < 2; ++phase)
    if (pending[phase] && (phase_q_tile_sizes[phase] < 1 ||
                           !range_ok(phase_node_offsets[phase], phase_node_nums[phase], num_kv_heads)))
      return FT_ERR_ARGUMENT;
  const bool narrow[2] = {is_narrow(phase_q_tile_sizes[0], g), is_narrow(phase_q_tile_sizes[1], g)};
  auto assign = [](Stage1Args& t, bool is_narrow_range, int begin, int count) {
    if (is_narrow_range) { t.narrow_begin = begin; t.narrow_count = count; }
    else { t.vnode_begin = begin; t.vnode_count = count; }
  };
  const int64_t widest_tile = std::max(narrow[0] ? 0 : phase_q_tile_sizes[0], narrow[1] ? 0 : phase_q_tile_sizes[1]);
  a.wide_rows = (int)std::min<int64_t>(widest_tile * g, 1 << 20);
  // Both phases go into one launch when one is wide and the other narrow, or when they are of
  // the same kind and adjacent in the vnode list (the planner's lists always are).
  if (pending[0] && pending[1] && narrow[0] == narrow[1]) {
    if (phase_node_offsets[0] + phase_node_nums[0] == phase_node_offsets[1] &&
        range_ok(phase_node_offsets[0], phase_node_nums[0] + phase_node_nums[1], num_kv_heads)) {
      assign(a, narrow[0], phase_node_offsets[0], phase_node_nums[0] + phase_node_nums[1]);
      return launch_stage1<false>(a, head_dim, dtype, stream);
    }
    for (int phase = 0; phase < 2; ++phase) {
      Stage1Args b = a;
      assign(b, narrow[phase], phase_node_offsets[phase], phase_node_nums[phase]);
      if (int rc = launch_stage1<false>(b, head_dim, dtype, stream)) return rc;
    }
    return FT_OK;
  }
  for (int phase = 0; phase < 2; ++phase)
    if (pending[phase]) assign(a, narrow[phase], phase_node_offsets[phase], phase_node_nums[phase]);
  return launch_stage1<false>(a, head_dim, dtype, stream);
}

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
                       float sm_scale, int dtype, ft_stream_t stream) {
  if (!phase_node_nums || !phase_node_offsets) return FT_ERR_NULL_POINTER;
  if (num_kv_heads < 1 || num_qo_heads % num_kv_heads != 0) return FT_ERR_GROUP;
  const int g = num_qo_heads / num_kv_heads;
  if (int rc = check_common(head_dim, g, dtype)) return rc;
  if (head_dim < 32) return FT_ERR_HEAD_DIM;  // the program table is for the direct-load kernels
  if (phase_node_nums[0] == 0 && phase_node_nums[1] == 0) return FT_OK;
  Stage1Args a;
  if (int rc = stage1_setup(a, q, k, v, sq0, sq1, sk0, sk1, sv0, sv1, vnode_to_kv_entries, vnode_to_kv_offs,
                            vnode_to_kv_lens, vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens, num_kv_heads, g,
                            head_dim, sm_scale, mid_o, so0, so1, mid_lse, sl0, dtype))
    return rc;
  for (int phase = 0; phase < 2; ++phase)
    if (!range_ok(phase_node_offsets[phase], phase_node_nums[phase], num_kv_heads)) return FT_ERR_ARGUMENT;
  if (num_programs < 0 || (int64_t)num_programs * num_kv_heads > INT32_MAX) return FT_ERR_ARGUMENT;
  if (num_programs > 0 && !prog_table) return FT_ERR_NULL_POINTER;
  if (narrow_in_programs < 0 || narrow_in_programs > phase_node_nums[1]) return FT_ERR_ARGUMENT;
  if (num_programs == 0 && (phase_node_nums[0] > 0 || narrow_in_programs > 0)) return FT_ERR_ARGUMENT;
  a.vnode_begin = phase_node_offsets[0]; a.vnode_count = phase_node_nums[0];
  a.narrow_begin = phase_node_offsets[1]; a.narrow_count = phase_node_nums[1];
  if (num_programs > 0) { a.prog_table = prog_table; a.num_programs = num_programs; a.narrow_in_programs = narrow_in_programs; }
  a.narrow_table = narrow_table;
  a.prog_records = num_programs > 0 ? prog_records : nullptr;
  a.wide_rows = kWideRows;
  return launch_stage1<false>(a, head_dim, dtype, stream);
}

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
                       float sm_scale, int dtype, ft_stream_t stream) {
  if (int rc = ft_stage1_programs(q, k, v, sq0, sq1, sk0, sk1, sv0, sv1, vnode_to_kv_entries, vnode_to_kv_offs,
                                  vnode_to_kv_lens, vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens, mid_o, so0,
                                  so1, mid_lse, sl0, phase_node_nums, phase_node_offsets, prog_table, num_programs,
                                  narrow_in_programs, narrow_table, prog_records, num_qo_heads, num_kv_heads, head_dim,
                                  sm_scale, dtype, stream))
    return rc;
  return stage2_with_table(req_to_vnode_entries, req_to_vnode_offs, req_to_vnode_lens, req_table, mid_o, so0, so1,
                           mid_lse, sl0, o, oo0, oo1, batch_size, num_qo_heads, head_dim, dtype, stream);
}

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
                     float sm_scale, int dtype, ft_stream_t stream) {
  if (num_rows < 0 || num_qo_heads < 1 || head_dim < 1) return FT_ERR_ARGUMENT;
  // mid_o: num_rows x num_qo_heads x head_dim floats, then (256-byte aligned) mid_lse: num_rows x num_qo_heads
  const unsigned __int128 o_bytes = (unsigned __int128)num_rows * (unsigned)num_qo_heads * (unsigned)head_dim * 4u;
  const unsigned __int128 lse_at = (o_bytes + 255u) / 256u * 256u;
  const unsigned __int128 need = lse_at + (unsigned __int128)num_rows * (unsigned)num_qo_heads * 4u;
  if (need > (unsigned __int128)FT_STATIC_SCRATCH_BYTES) return FT_ERR_SCRATCH;
  char* base = nullptr;
  if (int rc = static_scratch_of_current_device(&base)) return rc;
  float* mid_o = reinterpret_cast<float*>(base);
  float* mid_lse = reinterpret_cast<float*>(base + (size_t)lse_at);
  return ft_decode_programs(q, k, v, o, sq0, sq1, sk0, sk1, sv0, sv1, oo0, oo1, vnode_to_kv_entries, vnode_to_kv_offs,
                            vnode_to_kv_lens, vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens, req_to_vnode_entries,
                            req_to_vnode_offs, req_to_vnode_lens, mid_o, (int64_t)num_qo_heads * head_dim, head_dim,
                            mid_lse, num_qo_heads, phase_node_nums, phase_node_offsets, prog_table, num_programs,
                            narrow_in_programs, narrow_table, prog_records, req_table, batch_size, num_qo_heads, num_kv_heads, head_dim,
                            sm_scale, dtype, stream);
}

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
              float sm_scale, int dtype, ft_stream_t stream) {
  if (int rc = ft_stage1_phases(q, k, v, sq0, sq1, sk0, sk1, sv0, sv1, vnode_to_kv_entries, vnode_to_kv_offs,
                                vnode_to_kv_lens, vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens, mid_o, so0, so1,
                                mid_lse, sl0, phase_node_nums, phase_node_offsets, phase_q_tile_sizes,
                                phase_kv_tile_sizes, num_qo_heads, num_kv_heads, head_dim, sm_scale, dtype, stream))
    return rc;
  return ft_stage2(req_to_vnode_entries, req_to_vnode_offs, req_to_vnode_lens, mid_o, so0, so1, mid_lse, sl0, o, oo0,
                   oo1, batch_size, num_qo_heads, head_dim, dtype, stream);
}

int ft_deft_stage1(const void* q, const void* k, const void* v,
                   int64_t sq0, int64_t sq1, int64_t sk0, int64_t sk1, int64_t sv0, int64_t sv1,
                   const int32_t* vnode_to_kv_entries, const int32_t* vnode_to_kv_offs,
                   const int32_t* vnode_to_kv_lens, const int32_t* vnode_to_q_entries,
                   const int32_t* vnode_to_q_offs, const int32_t* vnode_to_q_lens,
                   const int64_t* causalmask, const int32_t* causalmask_offset,
                   int subtree_num, int num_qo_heads, int num_kv_heads, int head_dim, int mask_len, float sm_scale,
                   float* mid_o, int64_t so0, int64_t so1, float* mid_lse, int64_t sl0,
                   int dtype, ft_stream_t stream) {
  if (num_kv_heads < 1 || num_qo_heads % num_kv_heads != 0) return FT_ERR_GROUP;
  const int g = num_qo_heads / num_kv_heads;
  if (int rc = check_common(head_dim, g, dtype)) return rc;
  if (head_dim < 32) return FT_ERR_HEAD_DIM;
  if (subtree_num == 0) return FT_OK;
  DeftArgs d{};
  if (int rc = stage1_setup(d.s, q, k, v, sq0, sq1, sk0, sk1, sv0, sv1, vnode_to_kv_entries, vnode_to_kv_offs,
                            vnode_to_kv_lens, vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens, num_kv_heads, g,
                            head_dim, sm_scale, mid_o, so0, so1, mid_lse, sl0, dtype))
    return rc;
  if (!causalmask || !causalmask_offset) return FT_ERR_NULL_POINTER;
  if (subtree_num < 0 || !range_ok(0, subtree_num, num_kv_heads)) return FT_ERR_ARGUMENT;
  // a power of two of at most 64 requests per mask word, and few enough words per token for the
  // 128 query rows a block serves at a time
  if (mask_len < 1 || mask_len > 64 || (mask_len & (mask_len - 1)) != 0) return FT_ERR_ARGUMENT;
  const int requests_per_pass = (kWideRows + g - 1) / g + 1;
  if ((requests_per_pass + mask_len - 1) / mask_len + 1 > kDeftMaskGroups) return FT_ERR_ARGUMENT;
  d.causalmask = causalmask;
  d.causalmask_offset = causalmask_offset;
  d.mask_len = mask_len;
  d.num_subtrees = subtree_num;
  return launch_deft(d, head_dim, dtype, stream);
}

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
                   int mask_len, float sm_scale, int dtype, ft_stream_t stream) {
  if (int rc = ft_deft_stage1(q, k, v, sq0, sq1, sk0, sk1, sv0, sv1, vnode_to_kv_entries, vnode_to_kv_offs,
                              vnode_to_kv_lens, vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens, causalmask,
                              causalmask_offset, subtree_num, num_qo_heads, num_kv_heads, head_dim, mask_len, sm_scale,
                              mid_o, so0, so1, mid_lse, sl0, dtype, stream))
    return rc;
  return ft_stage2(req_to_vnode_entries, req_to_vnode_offs, req_to_vnode_lens, mid_o, so0, so1, mid_lse, sl0, o, oo0,
                   oo1, batch_size, num_qo_heads, head_dim, dtype, stream);
}

int ft_gathered_decode(const void* q, const void* k_cache, const void* v_cache,
                       const int32_t* cache_seqlens, void* o,
                       int64_t sq0, int64_t sq1, int64_t oo0, int64_t oo1,
                       int batch_size, int max_seqlen, int num_qo_heads, int num_kv_heads,
                       int head_dim, int kv_split, float sm_scale,
                       float* mid_o, float* mid_lse, int dtype, ft_stream_t stream) {
  if (num_kv_heads < 1 || num_qo_heads % num_kv_heads != 0) return FT_ERR_GROUP;
  const int g = num_qo_heads / num_kv_heads;
  if (int rc = check_common(head_dim, g, dtype)) return rc;
  if (batch_size == 0) return FT_OK;
  if (!q || !k_cache || !v_cache || !cache_seqlens || !o || !mid_o || !mid_lse) return FT_ERR_NULL_POINTER;
  if (batch_size < 0 || max_seqlen < 1 || kv_split < 1 || num_kv_heads > 65535 || !(sm_scale > 0.f)) return FT_ERR_ARGUMENT;
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(mid_o) || !aligned16(o) ||
      (sq0 | sq1) % 8 != 0 || (oo0 | oo1) % 4 != 0)
    return FT_ERR_ALIGNMENT;
  const int nsplit = (max_seqlen + kv_split - 1) / kv_split;
  if ((int64_t)batch_size * nsplit > INT32_MAX) return FT_ERR_ARGUMENT;
  Stage1Args a{};
  a.q = static_cast<const char*>(q);
  a.k = static_cast<const char*>(k_cache);
  a.v = static_cast<const char*>(v_cache);
  a.sq0 = sq0; a.sq1 = sq1;
  a.sk0 = a.sv0 = (int64_t)num_kv_heads * head_dim;
  a.sk1 = a.sv1 = head_dim;
  if (is_narrow(1, g)) { a.narrow_begin = 0; a.narrow_count = batch_size * nsplit; }
  else { a.vnode_begin = 0; a.vnode_count = batch_size * nsplit; a.wide_rows = g; }
  a.g = g;
  a.hkv = num_kv_heads;
  a.real_dim = head_dim;
  a.scale_log2 = sm_scale * kLog2e;
  a.mid_o = mid_o; a.so0 = (int64_t)num_qo_heads * head_dim; a.so1 = head_dim;
  a.mid_lse = mid_lse; a.sl0 = num_qo_heads;
  a.cache_seqlens = cache_seqlens; a.max_seqlen = max_seqlen; a.kv_split = kv_split; a.nsplit = nsplit;
  if (int rc = launch_stage1<true>(a, head_dim, dtype, stream)) return rc;
  Stage2Args b{};
  b.mid_o = mid_o; b.so0 = a.so0; b.so1 = a.so1; b.mid_lse = mid_lse; b.sl0 = a.sl0;
  b.o = static_cast<char*>(o); b.oo0 = oo0; b.oo1 = oo1;
  b.batch = batch_size; b.hq = num_qo_heads; b.nsplit = nsplit;
  return launch_stage2(b, head_dim, dtype, stream);
}

int ft_store_kv(const void* k_new, const void* v_new, int64_t kn0, int64_t kn1, int64_t vn0, int64_t vn1,
                const void* out_cache_loc, int loc_is_int64, int num_tokens,
                void* k_pool, void* v_pool, int64_t sk0, int64_t sk1, int64_t sv0, int64_t sv1,
                int64_t num_slots, int num_kv_heads, int head_dim, int dtype, ft_stream_t stream) {
  if (dtype != FT_DTYPE_F16 && dtype != FT_DTYPE_BF16) return FT_ERR_DTYPE;
  if (head_dim < 8 || head_dim % 8 != 0 || head_dim > 1024) return FT_ERR_HEAD_DIM;
  if (num_tokens == 0) return FT_OK;
  if (!k_new || !v_new || !out_cache_loc || !k_pool || !v_pool) return FT_ERR_NULL_POINTER;
  if (num_tokens < 0 || num_kv_heads < 1 || num_kv_heads > 65535 || num_slots < 0) return FT_ERR_ARGUMENT;
  if (!aligned16(k_new) || !aligned16(v_new) || !aligned16(k_pool) || !aligned16(v_pool) ||
      (kn0 | kn1 | vn0 | vn1 | sk0 | sk1 | sv0 | sv1) % 8 != 0)
    return FT_ERR_ALIGNMENT;
  if (kn0 < 0 || kn1 < 0 || vn0 < 0 || vn1 < 0 || sk0 < 0 || sk1 < 0 || sv0 < 0 || sv1 < 0) return FT_ERR_ARGUMENT;
  StoreArgs a{};
  a.k_new = static_cast<const char*>(k_new); a.v_new = static_cast<const char*>(v_new);
  a.kn0 = kn0; a.kn1 = kn1; a.vn0 = vn0; a.vn1 = vn1;
  a.loc = out_cache_loc; a.loc_is_int64 = loc_is_int64 ? 1 : 0;
  a.k_pool = static_cast<char*>(k_pool); a.v_pool = static_cast<char*>(v_pool);
  a.sk0 = sk0; a.sk1 = sk1; a.sv0 = sv0; a.sv1 = sv1;
  a.num_slots = num_slots; a.tokens = num_tokens; a.hkv = num_kv_heads; a.chunks = head_dim / 8;
  const int64_t threads = (int64_t)num_tokens * num_kv_heads * a.chunks;
  const int64_t blocks = (threads + 255) / 256;
  if (blocks > INT32_MAX) return FT_ERR_ARGUMENT;
  hipLaunchKernelGGL(store_kv_kernel, dim3((unsigned)blocks, 1, 1), dim3(256, 1, 1), 0, stream, a);
  return hipGetLastError() == hipSuccess ? FT_OK : FT_ERR_LAUNCH;
}

}  // extern "C"
