// nn.Embedding on the DP-SGD hot path:
//   per-sample gradients      opacus/grad_sample/embedding.py:25-64
//   ghost-clipping norms      opacus/grad_sample/embedding_norm_sample.py:27-151
// Both need, per sample, the positions grouped by id. The reference sorts
// (row, id) pairs with torch.unique and scatters with atomics; here each sample
// gets a linked list per distinct id, built by integer comparisons only:
//   leader[t] = 1 iff no t' < t in the sample has the same id
//   next[t]   = the smallest t' > t with the same id, or -1
// A leader then walks its list in increasing t and sums the backprop rows in
// registers - a fixed order, no atomics, each row of b read exactly once. The
// sorted-unique view the reference exposes (unique pairs + inverse index) is
// derived from the same flags: rank[t] = number of distinct ids below ids[t].
//
// For samples of up to kSortMax positions the lists come from a sort: one block per sample
// sorts its (id, position) pairs in LDS (bitonic network, ties broken by position), after
// which equal ids are neighbours in increasing position. Longer samples take the pairwise
// scan (quadratic in T, no LDS limit).
//
// (Tried and dropped for the ghost norm: one streaming pass for sum_t |b_t|^2 plus corrections
// |sum b_t|^2 - sum |b_t|^2 for the ids that occur more than once. It reads the rows of repeated
// ids twice and handles them list by list: 1.5 us per repeated id and sample, where text has
// hundreds per sequence. Walking the lists reads every row once whatever the ids are.)
#include <climits>

#include "dpk_common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / DPK_WAVE;
constexpr int kIdTile = 2048;  // ids staged in LDS per step of the pairwise scan
constexpr int kLeadersPerBlock = 16;

struct EmbWs {
  int32_t* next;
  int32_t* leader;
  int32_t* rank;
  int32_t* count;  // [n] distinct ids per sample
  int64_t* base;   // [n + 1] exclusive prefix of count
  float* partials;
};

size_t ws_layout(int64_t n, int64_t T, int64_t D, void* ws, EmbWs* out) {
  const int64_t nt = n * T;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    size_t o = off;
    off += dpk_align_up(bytes, 256);
    return o;
  };
  const size_t o_next = take(nt * 4), o_leader = take(nt * 4), o_rank = take(nt * 4);
  const size_t o_count = take(n * 4), o_base = take((n + 1) * 8);
  const int64_t tch = dpk_cdiv(T, kLeadersPerBlock), dch = dpk_cdiv(D > 0 ? D : 1, kThreads * 4);
  const size_t o_part = take(n * tch * dch * 4);
  if (out && ws) {
    char* p = static_cast<char*>(ws);
    out->next = reinterpret_cast<int32_t*>(p + o_next);
    out->leader = reinterpret_cast<int32_t*>(p + o_leader);
    out->rank = reinterpret_cast<int32_t*>(p + o_rank);
    out->count = reinterpret_cast<int32_t*>(p + o_count);
    out->base = reinterpret_cast<int64_t*>(p + o_base);
    out->partials = reinterpret_cast<float*>(p + o_part);
  }
  return off;
}

// grid = n * ceil(T / 64); a block owns 64 consecutive positions t of one sample, lane
// <-> position, and its four waves each scan a quarter of every LDS-staged tile of the
// sample's id row (all lanes of a wave read the same address: a broadcast). The scan is
// branch-free so that the reads of an unrolled stretch are in flight together; the
// waves' findings (seen before? nearest later occurrence) meet in LDS.
constexpr int kLinkPositions = DPK_WAVE;

__global__ __launch_bounds__(kThreads) void emb_link_kernel(const int64_t* __restrict__ ids,
                                                             int64_t T, int64_t V, int blocks_per_sample,
                                                             int32_t* __restrict__ next,
                                                             int32_t* __restrict__ leader,
                                                             int32_t* __restrict__ flag) {
  __shared__ int64_t tile[kIdTile];
  __shared__ int32_t w_before[kWaves][kLinkPositions], w_next[kWaves][kLinkPositions];
  const int64_t sample = blockIdx.x / blocks_per_sample;
  const int32_t Ti = static_cast<int32_t>(T);
  const int lane = threadIdx.x & (DPK_WAVE - 1), wave = threadIdx.x / DPK_WAVE;
  const int32_t t = static_cast<int32_t>(blockIdx.x % blocks_per_sample) * kLinkPositions + lane;
  const int64_t* row = ids + sample * T;
  const bool live = t < Ti;
  const int64_t mine = live ? row[t] : 0;
  int32_t before = 0;  // an earlier position holds the same id
  int32_t nxt = Ti;    // first later position with the same id
  for (int32_t c0 = 0; c0 < Ti; c0 += kIdTile) {
    const int32_t c1 = c0 + kIdTile < Ti ? c0 + kIdTile : Ti;
    __syncthreads();
    for (int32_t i = c0 + threadIdx.x; i < c1; i += kThreads) tile[i - c0] = row[i];
    __syncthreads();
    const int32_t quarter = (c1 - c0 + kWaves - 1) / kWaves;
    const int32_t u0 = c0 + wave * quarter;
    const int32_t u1 = u0 + quarter < c1 ? u0 + quarter : c1;
#pragma unroll 8
    for (int32_t u = u0; u < u1; ++u) {
      const bool eq = tile[u - c0] == mine;
      before |= (eq && u < t) ? 1 : 0;
      const int32_t cand = (eq && u > t) ? u : Ti;
      nxt = cand < nxt ? cand : nxt;
    }
  }
  w_before[wave][lane] = before;
  w_next[wave][lane] = nxt;
  __syncthreads();
  if (wave == 0 && live) {
#pragma unroll
    for (int w = 1; w < kWaves; ++w) {
      before |= w_before[w][lane];
      nxt = w_next[w][lane] < nxt ? w_next[w][lane] : nxt;
    }
    next[sample * T + t] = nxt < Ti ? nxt : -1;
    leader[sample * T + t] = before ? 0 : 1;
    if (flag && V > 0 && (mine < 0 || mine >= V)) *flag = 1;
  }
}

// ---- lists by sorting: one block per sample, T <= kSortMax -------------------------------
constexpr int kSortMax = 4096;  // (id, position) pairs of 12 bytes: 48 KB of LDS

// next / leader as above; rank[t] = index of ids[t] among the sample's distinct ids in
// ascending order and count[sample] = number of distinct ids (both only when rank != NULL).
// flag (nullable): raised when an id lies outside [0, V) and V > 0.
//
// The sorting network runs on registers: thread t holds the E = np / 256 pairs with indices
// t E .. t E + E - 1. A compare-exchange at distance j stays inside the thread for j < E,
// meets the partner thread t ^ (j / E) of the same wave through a lane exchange for
// j < 64 E, and goes through LDS (two barriers) only for the few stages beyond that.
// Two element types: ids that all lie in [0, 2^51) - every vocabulary - are sorted as one
// 64-bit word, id << 12 | position (T <= 4096), a third of the instructions per comparison;
// any other ids as (id, position) pairs.
struct IdPos {
  int64_t key;
  int32_t pos;
  __device__ __forceinline__ bool less(const IdPos& y) const { return key < y.key || (key == y.key && pos < y.pos); }
  __device__ __forceinline__ IdPos from_lane(int src) const {
    IdPos o;
    const uint32_t lo = __builtin_amdgcn_ds_bpermute(src, static_cast<int>(static_cast<uint32_t>(key)));
    const uint32_t hi = __builtin_amdgcn_ds_bpermute(src, static_cast<int>(static_cast<uint32_t>(key >> 32)));
    o.key = static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
    o.pos = __builtin_amdgcn_ds_bpermute(src, pos);
    return o;
  }
  __device__ __forceinline__ void put(int64_t* k, int32_t* p, int at) const {
    k[at] = key;
    p[at] = pos;
  }
  static __device__ __forceinline__ IdPos get(const int64_t* k, const int32_t* p, int at) {
    IdPos o;
    o.key = k[at];
    o.pos = p[at];
    return o;
  }
};
struct Packed {
  uint64_t w;  // id << 12 | position
  __device__ __forceinline__ bool less(const Packed& y) const { return w < y.w; }
  __device__ __forceinline__ Packed from_lane(int src) const {
    Packed o;
    const uint32_t lo = __builtin_amdgcn_ds_bpermute(src, static_cast<int>(static_cast<uint32_t>(w)));
    const uint32_t hi = __builtin_amdgcn_ds_bpermute(src, static_cast<int>(static_cast<uint32_t>(w >> 32)));
    o.w = (static_cast<uint64_t>(hi) << 32) | lo;
    return o;
  }
  __device__ __forceinline__ void put(int64_t* k, int32_t*, int at) const { k[at] = static_cast<int64_t>(w); }
  static __device__ __forceinline__ Packed get(const int64_t* k, const int32_t*, int at) {
    Packed o;
    o.w = static_cast<uint64_t>(k[at]);
    return o;
  }
};

// Bitonic network over np = E * kThreads elements, thread t holding elements t E .. t E + E - 1.
// key / pos: exchange arrays of np entries for the stages whose partner is in another wave.
template <int E, class Elem>
__device__ __forceinline__ void bitonic_sort(Elem (&v)[E], int64_t* key, int32_t* pos) {
  constexpr int np = E * kThreads;
  const int tid = threadIdx.x;
#pragma unroll 1
  for (int k = 2; k <= np; k <<= 1) {
    // distances that reach another thread, largest first
#pragma unroll 1
    for (int j = k >> 1; j >= E && j > 0; j >>= 1) {
      const int d = j / E;  // partner thread = tid ^ d, same slot
      const bool lower = (tid & d) == 0;
      Elem o[E];
      if (d < DPK_WAVE) {
        // all lane exchanges of the stage in flight before the first comparison
        const int src = ((tid & (DPK_WAVE - 1)) ^ d) << 2;
#pragma unroll
        for (int e = 0; e < E; ++e) o[e] = v[e].from_lane(src);
      } else {
        __syncthreads();  // earlier readers of the exchange arrays are done
#pragma unroll
        for (int e = 0; e < E; ++e) v[e].put(key, pos, e * kThreads + tid);
        __syncthreads();
#pragma unroll
        for (int e = 0; e < E; ++e) o[e] = Elem::get(key, pos, e * kThreads + (tid ^ d));
      }
#pragma unroll
      for (int e = 0; e < E; ++e) {
        const bool up = ((tid * E + e) & k) == 0;
        // the lower index keeps the smaller element of an ascending pair
        if (o[e].less(v[e]) == (lower == up)) v[e] = o[e];
      }
    }
    // distances inside the thread's own E elements (compile-time, so that v stays in registers)
#pragma unroll
    for (int j = E >> 1; j > 0; j >>= 1) {
      if (j >= k) continue;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        if ((e & j) != 0) continue;  // the pair (e, e + j) once
        const bool up = ((tid * E + e) & k) == 0;
        const Elem lo = v[e], hi = v[e | j];
        const bool swap = hi.less(lo) == up;
        v[e] = swap ? hi : lo;
        v[e | j] = swap ? lo : hi;
      }
    }
  }
}

template <int E>
struct SortMem {
  int64_t key[E * kThreads];
  int32_t pos[E * kThreads];
  int32_t runs[kThreads];
  int32_t wide;  // some id of the sample does not fit the packed form
};

// total: ids holds this many entries in all (the last "sample" may be shorter than T: a run of
// positions of a flattened batch). sorted_ids / sorted_pos (nullable): the sample's sorted (id,
// position) pairs, entry i of sample s at s * T + i, for a merge across samples.
template <int E>
__device__ __forceinline__ void sort_link_sample(SortMem<E>& m, int64_t sample, const int64_t* __restrict__ ids, int T,
                                                 int64_t V, int32_t* __restrict__ next, int32_t* __restrict__ leader,
                                                 int32_t* __restrict__ rank, int32_t* __restrict__ count,
                                                 int32_t* __restrict__ flag, int64_t total = INT64_MAX,
                                                 int64_t* __restrict__ sorted_ids = nullptr,
                                                 int32_t* __restrict__ sorted_pos = nullptr) {
  constexpr int64_t kPackLimit = int64_t{1} << 51;
  int64_t* key = m.key;
  int32_t* pos = m.pos;
  int32_t* runs = m.runs;
  int32_t& wide = m.wide;
  const int64_t* row = ids + sample * T;
  // entries of this sample (a short last run of a flattened batch: what lies past it is padding)
  const int len = total - sample * T < T ? static_cast<int>(total - sample * T) : T;
  const int tid = threadIdx.x;
  if (tid == 0) wide = 0;
  __syncthreads();
  IdPos v[E];
  bool bad = false, big = false;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int i = tid * E + e;
    const bool live = i < len;
    v[e].key = live ? row[i] : INT64_MAX;
    v[e].pos = live ? i : T + i;  // padding sorts behind every real pair, whatever its id (positions < T are real)
    bad = bad || (live && V > 0 && (v[e].key < 0 || v[e].key >= V));
    big = big || (live && (v[e].key < 0 || v[e].key >= kPackLimit));
  }
  if (bad && flag) *flag = 1;
  if (big) wide = 1;
  __syncthreads();
  if (wide) {
    bitonic_sort<E, IdPos>(v, key, pos);
  } else {
    Packed w[E];
#pragma unroll
    for (int e = 0; e < E; ++e)  // real words stay below 2^63; padding lies above, behind every real id
      w[e].w = v[e].pos < T ? (static_cast<uint64_t>(v[e].key) << 12) | static_cast<uint32_t>(v[e].pos)
                            : (uint64_t{1} << 63) + static_cast<uint32_t>(v[e].pos);
    bitonic_sort<E, Packed>(w, key, pos);
#pragma unroll
    for (int e = 0; e < E; ++e) {
      v[e].key = static_cast<int64_t>(w[e].w >> 12);
      v[e].pos = static_cast<int32_t>(w[e].w & 0xfffu);
    }
  }
  // sorted: equal ids are neighbours, positions ascending inside a run
  __syncthreads();
#pragma unroll
  for (int e = 0; e < E; ++e) {
    key[tid * E + e] = v[e].key;
    pos[tid * E + e] = v[e].pos;
  }
  __syncthreads();
  const int lo = tid * E, hi = lo + E < len ? lo + E : len;
  if (sorted_ids) {  // uniform
    for (int i = lo; i < hi; ++i) {
      sorted_ids[sample * T + i] = key[i];
      sorted_pos[sample * T + i] = pos[i];
    }
  }
  int32_t mine = 0;
  for (int i = lo; i < hi; ++i) {
    const bool lead = i == 0 || key[i - 1] != key[i];
    mine += lead ? 1 : 0;
    const int p = pos[i];
    next[sample * T + p] = (i + 1 < len && key[i + 1] == key[i]) ? pos[i + 1] : -1;
    leader[sample * T + p] = lead ? 1 : 0;
  }
  if (!rank) return;  // uniform
  runs[tid] = mine;
  __syncthreads();
  int32_t before = 0;
  for (int t = 0; t < tid; ++t) before += runs[t];
  for (int i = lo; i < hi; ++i) {
    if (i == 0 || key[i - 1] != key[i]) ++before;
    rank[sample * T + pos[i]] = before - 1;
  }
  if (tid == kThreads - 1) count[sample] = before;
}

template <int E>
__global__ __launch_bounds__(kThreads) void emb_sort_link_kernel(const int64_t* __restrict__ ids, int T, int64_t V,
                                                                  int32_t* __restrict__ next,
                                                                  int32_t* __restrict__ leader,
                                                                  int32_t* __restrict__ rank,
                                                                  int32_t* __restrict__ count,
                                                                  int32_t* __restrict__ flag) {
  __shared__ SortMem<E> m;
  sort_link_sample<E>(m, blockIdx.x, ids, T, V, next, leader, rank, count, flag);
}

// ---- lists across a whole batch: sorted runs, then a merge by binary search ------------------
// The L positions of a flattened batch are cut into runs of R <= kSortMax positions; one block
// sorts each run (the kernel above, which also leaves the run's sorted (id, position) pairs),
// and the kernel below links equal ids across runs: a position's successor is the next entry of
// its run when that has the same id, else the first entry with that id of the nearest later run
// that has one; it leads its list when no earlier entry of its run and no earlier run has the id.
// Lists are therefore in increasing position, as a single scan over the batch would build them.
template <int E>
__global__ __launch_bounds__(kThreads) void emb_sort_runs_kernel(const int64_t* __restrict__ ids, int R, int64_t V,
                                                                  int64_t total, int32_t* __restrict__ next,
                                                                  int32_t* __restrict__ leader,
                                                                  int64_t* __restrict__ sorted_ids,
                                                                  int32_t* __restrict__ sorted_pos,
                                                                  int32_t* __restrict__ flag) {
  __shared__ SortMem<E> m;
  sort_link_sample<E>(m, blockIdx.x, ids, R, V, next, leader, nullptr, nullptr, flag, total, sorted_ids, sorted_pos);
}

// One thread per sorted entry (run r, index i). The searches of a group of eight other runs advance
// together, so that eight loads are in flight per step instead of one.
__global__ __launch_bounds__(kThreads) void emb_merge_runs_kernel(const int64_t* __restrict__ sorted_ids,
                                                                   const int32_t* __restrict__ sorted_pos, int R,
                                                                   int64_t total, int nruns,
                                                                   int32_t* __restrict__ next,
                                                                   int32_t* __restrict__ leader) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int r = static_cast<int>(e / R), i = static_cast<int>(e % R);
  auto run_len = [&](int q) { return static_cast<int>(total - static_cast<int64_t>(q) * R < R ? total - static_cast<int64_t>(q) * R : R); };
  if (r >= nruns || i >= run_len(r)) return;
  const int64_t* mine = sorted_ids + static_cast<int64_t>(r) * R;
  const int64_t sid = mine[i];
  const int len = run_len(r);
  const bool first = i == 0 || mine[i - 1] != sid;
  const bool last = i + 1 == len || mine[i + 1] != sid;
  const int64_t g = static_cast<int64_t>(r) * R + sorted_pos[static_cast<int64_t>(r) * R + i];
  int64_t succ = last ? -1 : static_cast<int64_t>(r) * R + sorted_pos[static_cast<int64_t>(r) * R + i + 1];
  bool earlier = false;
  int best = nruns;
  if (first || last) {
    constexpr int G = 8;
    for (int q0 = 0; q0 < nruns; q0 += G) {
      int lo[G], left[G];
#pragma unroll
      for (int j = 0; j < G; ++j) {
        const int q = q0 + j;
        const bool want = q < nruns && ((q > r && last && q < best) || (q < r && first && !earlier));
        lo[j] = 0;
        left[j] = want ? run_len(q) : 0;
      }
      // lower bound of sid in every wanted run: at most 13 halvings of 4096 entries
#pragma unroll 1
      for (int step = 0; step < 13; ++step) {
#pragma unroll
        for (int j = 0; j < G; ++j) {
          if (left[j] > 0) {
            const int half = left[j] >> 1, mid = lo[j] + half;
            const int64_t v = sorted_ids[static_cast<int64_t>(q0 + j) * R + mid];
            if (v < sid) {
              lo[j] = mid + 1;
              left[j] -= half + 1;
            } else {
              left[j] = half;
            }
          }
        }
      }
#pragma unroll
      for (int j = 0; j < G; ++j) {
        const int q = q0 + j;
        const bool want = q < nruns && ((q > r && last && q < best) || (q < r && first && !earlier));
        if (want && lo[j] < run_len(q) && sorted_ids[static_cast<int64_t>(q) * R + lo[j]] == sid) {
          if (q > r) {
            best = q;
            succ = static_cast<int64_t>(q) * R + sorted_pos[static_cast<int64_t>(q) * R + lo[j]];
          } else {
            earlier = true;
          }
        }
      }
    }
  }
  next[g] = static_cast<int32_t>(succ);
  leader[g] = first && !earlier ? 1 : 0;
}

// rank[t] = #{leaders t' of the sample with ids[t'] < ids[t]}; count[sample] = #leaders.
__global__ __launch_bounds__(kThreads) void emb_rank_kernel(const int64_t* __restrict__ ids, int64_t T,
                                                             int blocks_per_sample,
                                                             const int32_t* __restrict__ leader,
                                                             int32_t* __restrict__ rank,
                                                             int32_t* __restrict__ count) {
  __shared__ int64_t tile[kIdTile];
  __shared__ int32_t lead[kIdTile];
  const int64_t sample = blockIdx.x / blocks_per_sample;
  const int bps = static_cast<int>(blockIdx.x % blocks_per_sample);
  const int64_t t = static_cast<int64_t>(bps) * kThreads + threadIdx.x;
  const int64_t* row = ids + sample * T;
  const int32_t* lrow = leader + sample * T;
  const bool live = t < T;
  const int64_t mine = live ? row[t] : 0;
  int32_t below = 0, total = 0;
  for (int64_t c0 = 0; c0 < T; c0 += kIdTile) {
    const int64_t cn = (T - c0 < kIdTile) ? T - c0 : kIdTile;
    __syncthreads();
    for (int64_t i = threadIdx.x; i < cn; i += kThreads) {
      tile[i] = row[c0 + i];
      lead[i] = lrow[c0 + i];
    }
    __syncthreads();
    for (int64_t i = 0; i < cn; ++i) {
      total += lead[i];
      if (lead[i] && tile[i] < mine) ++below;
    }
  }
  if (live) rank[sample * T + t] = below;
  if (bps == 0 && threadIdx.x == 0) count[sample] = total;
}

// One block: base = exclusive prefix of count over samples (sequential: n is a batch size).
__global__ void emb_prefix_kernel(const int32_t* __restrict__ count, int64_t n,
                                  int64_t* __restrict__ base, int64_t* __restrict__ n_unique) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  int64_t acc = 0;
  for (int64_t i = 0; i < n; ++i) {
    base[i] = acc;
    acc += count[i];
  }
  base[n] = acc;
  *n_unique = acc;
}

__global__ __launch_bounds__(kThreads) void emb_emit_pairs_kernel(
    const int64_t* __restrict__ ids, int64_t n, int64_t T, const int32_t* __restrict__ leader,
    const int32_t* __restrict__ rank, const int64_t* __restrict__ base, int64_t* __restrict__ inverse,
    int64_t* __restrict__ pairs) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n * T) return;
  const int64_t sample = i / T;
  const int64_t pos = base[sample] + rank[i];
  inverse[i] = pos;
  if (leader[i]) {
    pairs[2 * pos] = sample;
    pairs[2 * pos + 1] = ids[i];
  }
}

// grid = n * tch * dch. A block owns kLeadersPerBlock positions and 1024 columns;
// thread <-> 4 columns. MODE 0: sum of squares of the per-id sums (ghost norm).
// MODE 1: write scale * sum into gs[sample, id, :].
// MODE 2: as MODE 1 with every row multiplied by its weight rw[t] before it is added (the
// clip-weighted sum over a whole batch laid out as one "sample" of n * T positions).
template <typename TIN, typename TOUT, int MODE, bool VEC>
__global__ __launch_bounds__(kThreads) void emb_walk_kernel(
    const int64_t* __restrict__ ids, const TIN* __restrict__ b, const int32_t* __restrict__ next,
    const int32_t* __restrict__ leader, int64_t T, int64_t D, int64_t V, int tch, int dch,
    float scale, float* __restrict__ partials, TOUT* __restrict__ gs, const float* __restrict__ rw = nullptr) {
  __shared__ float red[kWaves];
  int64_t bid = blockIdx.x;
  const int dc = static_cast<int>(bid % dch);
  bid /= dch;
  const int tc = static_cast<int>(bid % tch);
  const int64_t sample = bid / tch;
  const int64_t d = (static_cast<int64_t>(dc) * kThreads + threadIdx.x) * 4;
  const int64_t t0 = static_cast<int64_t>(tc) * kLeadersPerBlock;
  const int64_t t1 = (t0 + kLeadersPerBlock < T) ? t0 + kLeadersPerBlock : T;
  const TIN* bs = b + sample * T * D;
  const int32_t* nx = next + sample * T;
  const int32_t* ld = leader + sample * T;
  float ss = 0.f;
  // the first row of every list that starts in this block is requested before any is used
  // (kLeadersPerBlock independent loads in flight); further members follow list by list
  // Everything a block needs first is requested without a branch in between, so that the
  // requests overlap: the list flags and second members of its positions (clamped reads, the
  // values past the end unused), then the first row of every list that starts here (other
  // positions re-read the block's first row, a cache hit). Further members follow list by list.
  typename dpk_io<TIN>::raw4 first[kLeadersPerBlock];
  int32_t head[kLeadersPerBlock], follow[kLeadersPerBlock];
#pragma unroll
  for (int r = 0; r < kLeadersPerBlock; ++r) {
    const int64_t t = (t0 + r < T) ? t0 + r : T - 1;
    head[r] = ld[t];
    follow[r] = nx[t];
  }
#pragma unroll
  for (int r = 0; r < kLeadersPerBlock; ++r)
    if (t0 + r >= t1 || !head[r]) follow[r] = -2;  // < -1: no list starts here
  if (VEC) {
    const int64_t dd = (d < D) ? d : 0;
#pragma unroll
    for (int r = 0; r < kLeadersPerBlock; ++r)
      first[r] = dpk_io<TIN>::load4_raw(bs + (follow[r] >= -1 ? t0 + r : t0) * D + dd);
  }
#pragma unroll
  for (int r = 0; r < kLeadersPerBlock; ++r) {
    const int64_t t = t0 + r;
    if (follow[r] < -1) continue;  // uniform over the block
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (VEC && d < D) {
      acc = dpk_io<TIN>::unpack4(first[r]);
      if (MODE == 2) {
        const float c = rw[t];
        acc.x *= c;
        acc.y *= c;
        acc.z *= c;
        acc.w *= c;
      }
    }
    if (d < D) {
      for (int64_t u = VEC ? static_cast<int64_t>(follow[r]) : t; u >= 0; u = nx[u]) {
        const TIN* p = bs + u * D + d;
        const float c = MODE == 2 ? rw[u] : 1.f;
        if (VEC) {
          const float4 v = dpk_io<TIN>::load4(p);
          acc.x = fmaf(c, v.x, acc.x);
          acc.y = fmaf(c, v.y, acc.y);
          acc.z = fmaf(c, v.z, acc.z);
          acc.w = fmaf(c, v.w, acc.w);
        } else {
          acc.x = fmaf(c, dpk_io<TIN>::load(p), acc.x);
          if (d + 1 < D) acc.y = fmaf(c, dpk_io<TIN>::load(p + 1), acc.y);
          if (d + 2 < D) acc.z = fmaf(c, dpk_io<TIN>::load(p + 2), acc.z);
          if (d + 3 < D) acc.w = fmaf(c, dpk_io<TIN>::load(p + 3), acc.w);
        }
      }
    }
    if (MODE == 0) {
      ss += (acc.x * acc.x + acc.y * acc.y) + (acc.z * acc.z + acc.w * acc.w);
    } else if (d < D) {
      const int64_t id = ids[sample * T + t];
      if (id >= 0 && id < V) {
        TOUT* o = gs + (sample * V + id) * D + d;
        acc.x *= scale;
        acc.y *= scale;
        acc.z *= scale;
        acc.w *= scale;
        if (VEC) {
          dpk_io<TOUT>::store4(o, acc);
        } else {
          dpk_io<TOUT>::store(o, acc.x);
          if (d + 1 < D) dpk_io<TOUT>::store(o + 1, acc.y);
          if (d + 2 < D) dpk_io<TOUT>::store(o + 2, acc.z);
          if (d + 3 < D) dpk_io<TOUT>::store(o + 3, acc.w);
        }
      }
    }
  }
  if (MODE == 0) {
    const float s = block_sum<kWaves>(ss, red);
    if (threadIdx.x == 0) partials[blockIdx.x] = s;
  }
}

// Zero fill with 16-byte stores (a kernel rather than a memset node, so that a
// caller may capture the stream into a graph).
__global__ __launch_bounds__(kThreads) void zero_fill_kernel(uint4* __restrict__ p, int64_t n16,
                                                              unsigned char* __restrict__ tail,
                                                              int64_t ntail) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n16; i += stride)
    p[i] = make_uint4(0u, 0u, 0u, 0u);
  if (blockIdx.x == 0 && threadIdx.x < ntail) tail[threadIdx.x] = 0;
}

// ---- EmbeddingBag ---------------------------------------------------------------
// *flag = 1 when an index lies outside [0, V), an offset outside [0, L] or the
// offsets decrease (never cleared here: the flag is the caller's and sticky).
__global__ __launch_bounds__(kThreads) void bag_check_kernel(const int64_t* __restrict__ index,
                                                              const int64_t* __restrict__ offsets,
                                                              int64_t L, int64_t nbags, int64_t V,
                                                              int32_t* __restrict__ flag) {
  const int64_t j = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  bool bad = false;
  if (j < L) bad = index[j] < 0 || index[j] >= V;
  if (j < nbags) {
    const int64_t o = offsets[j];
    bad = bad || o < 0 || o > L || (j + 1 < nbags && offsets[j + 1] < o);
  }
  if (bad) *flag = 1;
}

// One block per position j of the flat index list: finds the bag i that holds j
// (last i with offsets[i] <= j) and writes b[i,:] (divided by the bag length in mean
// mode) to gs[i, index[j], :]. Positions of one bag that repeat an index write the
// same values to the same row, so the row holds b[i,:] once however often the index
// occurs: the result of the reference's indexed "+=" (embedding.py:84-87).
template <typename TIN, typename TOUT>
__global__ __launch_bounds__(kThreads) void bag_scatter_kernel(
    const int64_t* __restrict__ index, const int64_t* __restrict__ offsets, const TIN* __restrict__ b,
    TOUT* __restrict__ gs, int64_t L, int64_t nbags, int64_t V, int64_t D, int mean, float scale) {
  const int64_t j = blockIdx.x;
  int64_t lo = 0, hi = nbags - 1;
  if (offsets[0] > j) return;  // before the first bag: belongs to none
  while (lo < hi) {
    const int64_t mid = (lo + hi + 1) >> 1;
    if (offsets[mid] <= j) lo = mid;
    else hi = mid - 1;
  }
  const int64_t bag = lo;
  const int64_t end = bag + 1 < nbags ? offsets[bag + 1] : L;
  const float len = static_cast<float>(end - offsets[bag]);
  const int64_t row = index[j];
  if (row < 0 || row >= V) return;  // reported by bag_check_kernel; nothing is written
  const TIN* src = b + bag * D;
  TOUT* dst = gs + (bag * V + row) * D;
  for (int64_t d = threadIdx.x; d < D; d += kThreads) {
    float v = dpk_io<TIN>::load(src + d) * scale;
    if (mean) v = v / len;
    dpk_io<TOUT>::store(dst + d, v);
  }
}

int check_common(const char* who, const int64_t* ids, int64_t n, int64_t T, int64_t D, void* ws,
                 size_t ws_bytes, EmbWs* w) {
  DPK_REQUIRE(ids, DPK_E_ARG, "%s: ids is NULL", who);
  DPK_REQUIRE(dpk_aligned(ids, 8), DPK_E_ALIGN, "%s: ids misaligned", who);
  DPK_REQUIRE(T < (1LL << 31) && n * dpk_cdiv(T, kLinkPositions) <= DPK_MAX_GRID_X, DPK_E_SHAPE,
              "%s: n=%lld T=%lld too large", who, (long long)n, (long long)T);
  const size_t need = ws_layout(n, T, D, nullptr, nullptr);
  DPK_REQUIRE(ws && ws_bytes >= need, DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes,
              need);
  DPK_REQUIRE(dpk_aligned(ws, 256), DPK_E_ALIGN, "%s: workspace must be 256-byte aligned", who);
  ws_layout(n, T, D, ws, w);
  return DPK_OK;
}

bool sorts_in_lds(int64_t n, int64_t T) { return T <= kSortMax && n <= DPK_MAX_GRID_X; }

// status: the caller's sticky flag (NULL: no range check), set when an id lies outside [0, V).
// with_rank: also fill w.rank and w.count (the sorting kernel does it in passing; after the
// pairwise scan the caller runs emb_rank_kernel). Returns whether the sorting kernel ran.
bool launch_link(const int64_t* ids, int64_t n, int64_t T, int64_t V, const EmbWs& w, int32_t* status,
                 bool with_rank, hipStream_t s) {
  if (sorts_in_lds(n, T)) {
    const dim3 grid(static_cast<unsigned>(n)), block(kThreads);
    int32_t* rk = with_rank ? w.rank : nullptr;
    int32_t* ct = with_rank ? w.count : nullptr;
    const int Ti = static_cast<int>(T);
#define DPK_SORT(E_) hipLaunchKernelGGL(emb_sort_link_kernel<E_>, grid, block, 0, s, ids, Ti, V, w.next, w.leader, rk, ct, status)
    if (T <= 256) DPK_SORT(1);
    else if (T <= 512) DPK_SORT(2);
    else if (T <= 1024) DPK_SORT(4);
    else if (T <= 2048) DPK_SORT(8);
    else DPK_SORT(16);
#undef DPK_SORT
    return true;
  }
  const int bps = static_cast<int>(dpk_cdiv(T, kLinkPositions));
  hipLaunchKernelGGL(emb_link_kernel, dim3(static_cast<unsigned>(n * bps)), dim3(kThreads), 0, s, ids, T,
                     V, bps, w.next, w.leader, status);
  return false;
}

template <typename TIN, typename TOUT, int MODE>
void launch_walk(bool vec, const int64_t* ids, const void* b, const EmbWs& w, int64_t n, int64_t T,
                 int64_t D, int64_t V, float scale, void* gs, hipStream_t s, const float* rw = nullptr) {
  const int tch = static_cast<int>(dpk_cdiv(T, kLeadersPerBlock));
  const int dch = static_cast<int>(dpk_cdiv(D, kThreads * 4));
  const dim3 grid(static_cast<unsigned>(n * tch * dch)), block(kThreads);
  if (vec)
    hipLaunchKernelGGL((emb_walk_kernel<TIN, TOUT, MODE, true>), grid, block, 0, s, ids,
                       static_cast<const TIN*>(b), w.next, w.leader, T, D, V, tch, dch, scale,
                       w.partials, static_cast<TOUT*>(gs), rw);
  else
    hipLaunchKernelGGL((emb_walk_kernel<TIN, TOUT, MODE, false>), grid, block, 0, s, ids,
                       static_cast<const TIN*>(b), w.next, w.leader, T, D, V, tch, dch, scale,
                       w.partials, static_cast<TOUT*>(gs), rw);
}

// rw[r] = coef[r / T]: the weight of position r of the flattened batch.
__global__ __launch_bounds__(kThreads) void emb_row_weights_kernel(const float* __restrict__ coef, float* __restrict__ rw,
                                                                     int64_t rows, int64_t T) {
  const int64_t r = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (r < rows) rw[r] = coef[r / T];
}

}  // namespace

extern "C" size_t dpk_embedding_workspace_bytes(int64_t n, int64_t T, int64_t D) {
  if (n <= 0 || T <= 0) return 0;
  return ws_layout(n, T, D, nullptr, nullptr);
}

extern "C" int dpk_embedding_unique_pairs(const int64_t* ids, int64_t n, int64_t T,
                                          int64_t* inverse, int64_t* unique_pairs,
                                          int64_t* n_unique, void* ws, size_t ws_bytes,
                                          dpk_stream_t stream) {
  const char* who = "dpk_embedding_unique_pairs";
  DPK_REQUIRE(n >= 0 && T >= 0, DPK_E_SHAPE, "%s: n=%lld T=%lld", who, (long long)n, (long long)T);
  if (n == 0 || T == 0) return DPK_OK;
  DPK_REQUIRE(inverse && unique_pairs && n_unique, DPK_E_ARG, "%s: NULL output", who);
  EmbWs w;
  int rc = check_common(who, ids, n, T, 0, ws, ws_bytes, &w);
  if (rc != DPK_OK) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool ranked = launch_link(ids, n, T, 0, w, nullptr, true, s);
  DPK_LAUNCH_CHECK(who);
  if (!ranked) {
    const int bps = static_cast<int>(dpk_cdiv(T, kThreads));
    hipLaunchKernelGGL(emb_rank_kernel, dim3(static_cast<unsigned>(n * bps)), dim3(kThreads), 0, s, ids, T,
                       bps, w.leader, w.rank, w.count);
  }
  hipLaunchKernelGGL(emb_prefix_kernel, dim3(1), dim3(64), 0, s, w.count, n, w.base, n_unique);
  hipLaunchKernelGGL(emb_emit_pairs_kernel, dim3(static_cast<unsigned>(dpk_cdiv(n * T, kThreads))),
                     dim3(kThreads), 0, s, ids, n, T, w.leader, w.rank, w.base, inverse, unique_pairs);
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}

extern "C" int dpk_embedding_ghost_norm(const int64_t* ids, const void* b, int dtype, float* norm,
                                        int64_t n, int64_t T, int64_t D, float scale, void* ws,
                                        size_t ws_bytes, dpk_stream_t stream) {
  const char* who = "dpk_embedding_ghost_norm";
  DPK_REQUIRE(n >= 0 && T >= 1 && D >= 1, DPK_E_SHAPE, "%s: n=%lld T=%lld D=%lld", who, (long long)n,
              (long long)T, (long long)D);
  if (n == 0) return DPK_OK;
  DPK_REQUIRE(b && norm, DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(dtype), DPK_E_DTYPE, "%s: dtype %d", who, dtype);
  DPK_REQUIRE(dpk_aligned(b, dpk_elsize(dtype)), DPK_E_ALIGN, "%s: misaligned tensor", who);
  EmbWs w;
  int rc = check_common(who, ids, n, T, D, ws, ws_bytes, &w);
  if (rc != DPK_OK) return rc;
  const int64_t tch = dpk_cdiv(T, kLeadersPerBlock), dch = dpk_cdiv(D, kThreads * 4);
  DPK_REQUIRE(n * tch * dch <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: too many blocks", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  launch_link(ids, n, T, 0, w, nullptr, false, s);
  DPK_LAUNCH_CHECK(who);
  const bool vec = D % 4 == 0 && dpk_aligned(b, dtype == DPK_BF16 ? 8 : 16);
  if (dtype == DPK_F32) launch_walk<float, float, 0>(vec, ids, b, w, n, T, D, 0, scale, nullptr, s);
  else launch_walk<bf16_t, float, 0>(vec, ids, b, w, n, T, D, 0, scale, nullptr, s);
  DPK_LAUNCH_CHECK(who);
  dpk_launch_reduce_rows(w.partials, n, tch * dch, norm, 1, fabsf(scale), s);
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}

extern "C" int dpk_embedding_gs(const int64_t* ids, const void* b, int in_dtype, void* gs,
                                int gs_dtype, int64_t n, int64_t T, int64_t V, int64_t D,
                                float scale, int32_t* status, void* ws, size_t ws_bytes,
                                dpk_stream_t stream) {
  const char* who = "dpk_embedding_gs";
  DPK_REQUIRE(n >= 0 && T >= 1 && V >= 1 && D >= 1, DPK_E_SHAPE, "%s: n=%lld T=%lld V=%lld D=%lld", who,
              (long long)n, (long long)T, (long long)V, (long long)D);
  if (n == 0) return DPK_OK;
  DPK_REQUIRE(b && gs, DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(in_dtype) && in_dtype == gs_dtype, DPK_E_DTYPE,
              "%s: dtypes %d,%d (must be equal)", who, in_dtype, gs_dtype);
  DPK_REQUIRE(dpk_aligned(b, dpk_elsize(in_dtype)) && dpk_aligned(gs, dpk_elsize(gs_dtype)),
              DPK_E_ALIGN, "%s: misaligned tensor", who);
  EmbWs w;
  int rc = check_common(who, ids, n, T, D, ws, ws_bytes, &w);
  if (rc != DPK_OK) return rc;
  const int64_t tch = dpk_cdiv(T, kLeadersPerBlock), dch = dpk_cdiv(D, kThreads * 4);
  DPK_REQUIRE(n * tch * dch <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: too many blocks", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  DPK_REQUIRE(dpk_aligned(status, 4), DPK_E_ALIGN, "%s: status misaligned", who);
  // Ids outside [0, V) would address memory outside gs: the walk below writes nothing for
  // them, and the link kernel raises the caller's flag.
  launch_link(ids, n, T, V, w, status, false, s);
  DPK_LAUNCH_CHECK(who);
  const size_t bytes = static_cast<size_t>(n) * V * D * dpk_elsize(gs_dtype);
  const int64_t n16 = dpk_aligned(gs, 16) ? static_cast<int64_t>(bytes / 16) : 0;
  const int64_t ntail = static_cast<int64_t>(bytes - static_cast<size_t>(n16) * 16);
  if (n16 > 0 || ntail > 0) {
    DPK_REQUIRE(ntail < kThreads, DPK_E_ALIGN, "%s: gs must be 16-byte aligned", who);
    int64_t blocks = dpk_cdiv(n16 > 0 ? n16 : 1, kThreads * 4);
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(zero_fill_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0, s,
                       static_cast<uint4*>(gs), n16,
                       static_cast<unsigned char*>(gs) + static_cast<size_t>(n16) * 16, ntail);
    DPK_LAUNCH_CHECK(who);
  }
  const bool vec = D % 4 == 0 && dpk_aligned(b, in_dtype == DPK_BF16 ? 8 : 16) &&
                   dpk_aligned(gs, gs_dtype == DPK_BF16 ? 8 : 16);
  if (in_dtype == DPK_F32) launch_walk<float, float, 1>(vec, ids, b, w, n, T, D, V, scale, gs, s);
  else launch_walk<bf16_t, bf16_t, 1>(vec, ids, b, w, n, T, D, V, scale, gs, s);
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}

namespace {
// Run length of the batch-wide sort: short runs sort faster and give more blocks, long runs keep the
// number of runs (searches per entry in the merge) down.
int batch_run_length(int64_t L) { return L <= 1024 ? static_cast<int>(L <= 256 ? 256 : (L <= 512 ? 512 : 1024)) : (L <= 32768 ? 1024 : kSortMax); }

struct EmbBatchLayout {
  size_t lists, weights, sorted_ids, sorted_pos, total;
};
EmbBatchLayout batch_layout(int64_t L, int64_t D) {
  EmbBatchLayout l;
  const int R = batch_run_length(L);
  const int64_t padded = dpk_cdiv(L, R) * R;
  l.lists = ws_layout(1, L, D, nullptr, nullptr);
  l.weights = l.lists;
  l.sorted_ids = l.weights + dpk_align_up(static_cast<size_t>(L) * sizeof(float), 256);
  l.sorted_pos = l.sorted_ids + dpk_align_up(static_cast<size_t>(padded) * sizeof(int64_t), 256);
  l.total = l.sorted_pos + dpk_align_up(static_cast<size_t>(padded) * sizeof(int32_t), 256);
  return l;
}
}  // namespace

extern "C" size_t dpk_embedding_weighted_sum_workspace_bytes(int64_t n, int64_t T, int64_t D) {
  if (n <= 0 || T <= 0) return 0;
  return batch_layout(n * T, D).total;
}

// out[v, :] = scale * sum_n coef[n] * sum_{t : ids[n,t] == v} b[n,t,:]: the clip-weighted sum of the
// per-sample gradients of an Embedding table (embedding.py:48-61 weighted per sample), what the
// second backward pass of sum_n coef[n] * loss[n] leaves in weight.grad
// (utils/fast_gradient_clipping_utils.py:193-201). The batch is taken as one run of n * T
// positions: equal ids are linked across samples, each list is summed in fp32 in position order
// with every row times its sample's coefficient, and a row of the table is written once. out is
// fully written (rows no id names are zero). Ids outside [0, V): as for dpk_embedding_gs.
extern "C" int dpk_embedding_weighted_sum(const int64_t* ids, const void* b, int in_dtype, const float* coef, void* out,
                                          int out_dtype, int64_t n, int64_t T, int64_t V, int64_t D, float scale,
                                          int32_t* status, void* ws, size_t ws_bytes, dpk_stream_t stream) {
  const char* who = "dpk_embedding_weighted_sum";
  DPK_REQUIRE(n >= 1 && T >= 1 && V >= 1 && D >= 1, DPK_E_SHAPE, "%s: n=%lld T=%lld V=%lld D=%lld", who, (long long)n,
              (long long)T, (long long)V, (long long)D);
  DPK_REQUIRE(b && coef && out, DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(in_dtype) && dpk_dtype_ok(out_dtype) && (in_dtype == out_dtype || out_dtype == DPK_F32),
              DPK_E_DTYPE, "%s: dtypes %d,%d (the result in the input's type or fp32)", who, in_dtype, out_dtype);
  DPK_REQUIRE(dpk_aligned(b, dpk_elsize(in_dtype)) && dpk_aligned(out, 16) && dpk_aligned(coef, 4) && dpk_aligned(status, 4),
              DPK_E_ALIGN, "%s: misaligned tensor (out must be 16-byte aligned)", who);
  const int64_t L = n * T;
  DPK_REQUIRE(L < (int64_t{1} << 31), DPK_E_SHAPE, "%s: n * T = %lld positions", who, (long long)L);
  const EmbBatchLayout lay = batch_layout(L, D);
  EmbWs w;
  int rc = check_common(who, ids, 1, L, D, ws, ws_bytes, &w);
  if (rc != DPK_OK) return rc;
  DPK_REQUIRE(ws_bytes >= lay.total, DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes, lay.total);
  char* base = static_cast<char*>(ws);
  float* rw = reinterpret_cast<float*>(base + lay.weights);
  int64_t* sorted_ids = reinterpret_cast<int64_t*>(base + lay.sorted_ids);
  int32_t* sorted_pos = reinterpret_cast<int32_t*>(base + lay.sorted_pos);
  const int64_t tch = dpk_cdiv(L, kLeadersPerBlock), dch = dpk_cdiv(D, kThreads * 4);
  const int R = batch_run_length(L);
  const int64_t nruns = dpk_cdiv(L, R);
  DPK_REQUIRE(tch * dch <= DPK_MAX_GRID_X && nruns <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: too many blocks", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(emb_row_weights_kernel, dim3(static_cast<unsigned>(dpk_cdiv(L, kThreads))), dim3(kThreads), 0, s, coef,
                     rw, L, T);
  // lists of equal ids over the whole batch: sorted runs, merged by binary search
  {
    const dim3 grid(static_cast<unsigned>(nruns)), block(kThreads);
#define DPK_RUNS(E_) \
  hipLaunchKernelGGL(emb_sort_runs_kernel<E_>, grid, block, 0, s, ids, R, V, L, w.next, w.leader, sorted_ids, sorted_pos, status)
    if (R <= 256) DPK_RUNS(1);
    else if (R <= 512) DPK_RUNS(2);
    else if (R <= 1024) DPK_RUNS(4);
    else DPK_RUNS(16);
#undef DPK_RUNS
    DPK_LAUNCH_CHECK(who);
    hipLaunchKernelGGL(emb_merge_runs_kernel, dim3(static_cast<unsigned>(dpk_cdiv(nruns * R, kThreads))), dim3(kThreads), 0,
                       s, sorted_ids, sorted_pos, R, L, static_cast<int>(nruns), w.next, w.leader);
  }
  DPK_LAUNCH_CHECK(who);
  const size_t bytes = static_cast<size_t>(V) * D * dpk_elsize(out_dtype);
  const int64_t n16 = static_cast<int64_t>(bytes / 16);
  const int64_t ntail = static_cast<int64_t>(bytes - static_cast<size_t>(n16) * 16);
  int64_t blocks = dpk_cdiv(n16 > 0 ? n16 : 1, kThreads * 4);
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(zero_fill_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0, s, static_cast<uint4*>(out),
                     n16, static_cast<unsigned char*>(out) + static_cast<size_t>(n16) * 16, ntail);
  DPK_LAUNCH_CHECK(who);
  const bool vec = D % 4 == 0 && dpk_aligned(b, in_dtype == DPK_BF16 ? 8 : 16);
  if (in_dtype == DPK_F32) launch_walk<float, float, 2>(vec, ids, b, w, 1, L, D, V, scale, out, s, rw);
  else if (out_dtype == DPK_BF16) launch_walk<bf16_t, bf16_t, 2>(vec, ids, b, w, 1, L, D, V, scale, out, s, rw);
  else launch_walk<bf16_t, float, 2>(vec, ids, b, w, 1, L, D, V, scale, out, s, rw);
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}

extern "C" int dpk_embedding_bag_gs(const int64_t* index, const int64_t* offsets, const void* b,
                                    int in_dtype, void* gs, int gs_dtype, int64_t nbags, int64_t L,
                                    int64_t V, int64_t D, int mean, float scale, int32_t* status,
                                    dpk_stream_t stream) {
  const char* who = "dpk_embedding_bag_gs";
  DPK_REQUIRE(nbags >= 0 && L >= 0 && V >= 1 && D >= 1, DPK_E_SHAPE, "%s: bags=%lld L=%lld V=%lld D=%lld",
              who, (long long)nbags, (long long)L, (long long)V, (long long)D);
  if (nbags == 0) return DPK_OK;
  DPK_REQUIRE(offsets && b && gs && (index || L == 0), DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(in_dtype) && in_dtype == gs_dtype, DPK_E_DTYPE,
              "%s: dtypes %d,%d (must be equal)", who, in_dtype, gs_dtype);
  DPK_REQUIRE(dpk_aligned(index, 8) && dpk_aligned(offsets, 8) && dpk_aligned(b, dpk_elsize(in_dtype)) &&
                  dpk_aligned(gs, 16),
              DPK_E_ALIGN, "%s: misaligned tensor (gs needs 16 bytes)", who);
  DPK_REQUIRE(dpk_aligned(status, 4), DPK_E_ALIGN, "%s: status misaligned", who);
  DPK_REQUIRE(L <= DPK_MAX_GRID_X && nbags <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: too many positions", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  // Bad indices would address memory outside gs: the scatter below writes nothing for them
  // (and reads b only inside [0, bags)), and the check kernel raises the caller's flag.
  if (status) {
    const int64_t most = L > nbags ? L : nbags;
    hipLaunchKernelGGL(bag_check_kernel, dim3(static_cast<unsigned>(dpk_cdiv(most, kThreads))), dim3(kThreads), 0,
                       s, index, offsets, L, nbags, V, status);
    DPK_LAUNCH_CHECK(who);
  }
  const size_t bytes = static_cast<size_t>(nbags) * V * D * dpk_elsize(gs_dtype);
  const int64_t n16 = static_cast<int64_t>(bytes / 16);
  const int64_t ntail = static_cast<int64_t>(bytes - static_cast<size_t>(n16) * 16);
  int64_t blocks = dpk_cdiv(n16 > 0 ? n16 : 1, kThreads * 4);
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(zero_fill_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0, s,
                     static_cast<uint4*>(gs), n16, static_cast<unsigned char*>(gs) + static_cast<size_t>(n16) * 16,
                     ntail);
  DPK_LAUNCH_CHECK(who);
  if (L > 0) {
    const dim3 grid(static_cast<unsigned>(L)), block(kThreads);
    if (in_dtype == DPK_F32)
      hipLaunchKernelGGL((bag_scatter_kernel<float, float>), grid, block, 0, s, index, offsets,
                         static_cast<const float*>(b), static_cast<float*>(gs), L, nbags, V, D, mean, scale);
    else
      hipLaunchKernelGGL((bag_scatter_kernel<bf16_t, bf16_t>), grid, block, 0, s, index, offsets,
                         static_cast<const bf16_t*>(b), static_cast<bf16_t*>(gs), L, nbags, V, D, mean, scale);
    DPK_LAUNCH_CHECK(who);
  }
  return DPK_OK;
}
