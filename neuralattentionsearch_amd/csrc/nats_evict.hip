// KV eviction + compaction of the NAtS layer caches (HBM-bound byte moves, bit exact).
//
// Follows NAtSChunkLayerCache._post_update (components/cache/nats_chunk_layer_cache.py:270-371), its
// helpers move_sliding_window_tokens_to_head (:391-437), get_updated_cache_info (:715-868),
// mask_invalid_tokens (:634-656) and merge_local_to_global_caches (components/cache/cache_update.py:25-76).
//
// plan kernels : a wavefront per (b, kv head) pulls the role slots into registers, marks the kept slots
//                (globals + locals after the last global) and gives each one its destination rank by a
//                wave-wide prefix sum (stream compaction of slot ids); one more workgroup folds the heads
//                into the global decisions and scalars.
// The per-token cache (params.update_chunk != 0; NAtSLayerCache._post_update, components/cache/nats_layer_cache.py:
// 292-418, with move_sliding_window_tokens_to_head :424-458, get_updated_cache_info :651-770 and mask_invalid_tokens
// :556-574) runs through the same kernels with one-token chunks: its sizes follow the same arithmetic; what differs
// is the ring (rows copied whatever the role, the slot after `tail` written first), that rows beyond the new
// n_ctx_data keep their contents, that a block of sliding-window tokens leaves n_ctx_data alone, and that a block
// completed by a one-token step takes the general path.
//
// apply kernels: move chunk-granular row blocks.  In place, a workgroup owns one row slice of every chunk
//                of one (b, kv head, tensor) and processes the ordered move list in batches, reading a
//                whole batch before writing it; because destinations never pass sources this equals
//                gather-everything-then-scatter.  Out of place (first prefill) every destination chunk is
//                produced independently straight from the raw K / V of the prefill.
#include "nats_common.h"

#include <stddef.h>

namespace nats {

struct HeadPlan {
  int32_t count;     // kept chunks (general path) or 1 (single completed chunk)
  int32_t dst_base;  // destination of the first kept chunk, in chunks
  int64_t sg_new;
  int64_t sl_new;
  int32_t all_sw;    // every slot of this head is sliding-window
  int32_t all_local; // every slot of this head is local
};

constexpr size_t kPlanHeaderBytes = 256;  // (its first word: the ticket counter of evict_plan_heads_kernel, zero between launches)

// The sizes a head brings into an eviction.  A cache that has seen nothing before these tokens (p.first) holds the
// empty ring and no local rows whatever its size tensors contain: they need not have been reset.
__device__ __forceinline__ long long old_size_global(const nats_evict_params& p, const int64_t* __restrict__ size_global, int h) {
  return p.first ? (long long)p.W : (long long)size_global[h];
}
__device__ __forceinline__ long long old_size_local(const nats_evict_params& p, const int64_t* __restrict__ size_local, int h) {
  return p.first ? 0LL : (long long)size_local[h];
}

// A one-token step that completes a chunk scatters that chunk for every head (nats_chunk_layer_cache.py:289-330); the
// per-token cache does the same with its one token when nothing is deferred (update_chunk_size == 1,
// nats_layer_cache.py:328-367), with the same arithmetic for the sizes.
__host__ __device__ inline bool one_step_scatter(const nats_evict_params& p) { return p.x_len == 1 && p.update_chunk <= 1; }

__host__ __device__ inline size_t plan_lists_offset(int64_t n_heads) {
  return (kPlanHeaderBytes + (size_t)n_heads * sizeof(HeadPlan) + 255) & ~size_t(255);
}

// ---------------------------------------------------------------------------------------------------
// plan, step 1: one wavefront per (b, kv head).  The head's role bytes are pulled into registers 1024
// slots at a time (16 per lane), so the scan costs one memory latency per block; ballots are replaced by
// per-lane bit masks plus wave-wide prefix sums, which give every kept slot its destination rank.
// ---------------------------------------------------------------------------------------------------
__device__ __forceinline__ int wave_sum(int x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
  return x;
}
__device__ __forceinline__ int wave_max(int x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x = max(x, __shfl_xor(x, o));
  return x;
}
__device__ __forceinline__ int wave_excl_scan(int x, int lane) {
  int incl = x;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    int y = __shfl_up(incl, o);
    if (lane >= o) incl += y;
  }
  return incl - x;
}

constexpr int kSlotsPerLane = 16;
constexpr int kSlotsPerBlock = kSlotsPerLane * kWave;

__device__ __forceinline__ void load_roles(const uint8_t* __restrict__ r, int S, int base, int lane, int* rb) {
#pragma unroll
  for (int j = 0; j < kSlotsPerLane; ++j) {
    int s = base + lane * kSlotsPerLane + j;
    rb[j] = s < S ? r[s] : 255;
  }
}

template <bool kCoherent = false>
__device__ __forceinline__ void plan_one_head(const uint8_t* __restrict__ roles, const int64_t* __restrict__ size_global,
                                              const int64_t* __restrict__ size_local, const nats_evict_params& p,
                                              char* __restrict__ ws, int head, int lane) {
  const int n_heads = (int)(p.B * p.H_kv);
  const int S = (int)p.S;
  const int C = (int)p.C;
  const int partial = (int)(p.fill % p.C);
  const int n_done = (int)(p.fill / p.C);
  const int S_eff = S - (partial ? 1 : 0);
  HeadPlan* plans = reinterpret_cast<HeadPlan*>(ws + kPlanHeaderBytes);
  int32_t* keep = reinterpret_cast<int32_t*>(ws + plan_lists_offset(n_heads)) + (int64_t)head * S;
  const uint8_t* r = roles + (int64_t)head * S;
  const long long sg = old_size_global(p, size_global, head), sl = old_size_local(p, size_local, head);
  HeadPlan hp;
  if (one_step_scatter(p)) {
    // one completed chunk is scattered for every head (:289-330)
    int r0 = r[0], rl = r[S - 1];
    bool is_g = r0 == NATS_ROLE_GLOBAL;
    long long dst = is_g ? sg : sg + sl;
    long long dec = (is_g ? sl / C + 1 : 0) + (rl == NATS_ROLE_SW ? 1 : 0);
    hp.count = 1;
    hp.dst_base = (int32_t)(dst / C);
    hp.sg_new = sg + (is_g ? C : 0);
    hp.sl_new = sl - dec * C + (long long)n_done * C;
    hp.all_sw = r0 == NATS_ROLE_SW;
    hp.all_local = 0;
    if (lane == 0) keep[0] = 0;
  } else {
    // pass 1: counts and the last complete global slot
    int n_glob_all = 0, n_sw = 0, n_loc = 0, last_g = -1;
    for (int base = 0; base < S; base += kSlotsPerBlock) {
      int rb[kSlotsPerLane];
      load_roles(r, S, base, lane, rb);
#pragma unroll
      for (int j = 0; j < kSlotsPerLane; ++j) {
        int s = base + lane * kSlotsPerLane + j;
        n_glob_all += rb[j] == NATS_ROLE_GLOBAL;
        n_sw += rb[j] == NATS_ROLE_SW;
        n_loc += rb[j] == NATS_ROLE_LOCAL;
        if (rb[j] == NATS_ROLE_GLOBAL && s < S_eff) last_g = s;
      }
    }
    n_glob_all = wave_sum(n_glob_all);
    n_sw = wave_sum(n_sw);
    n_loc = wave_sum(n_loc);
    last_g = wave_max(last_g);
    // pass 2: kept slots in order, destination rank by prefix sum (stream compaction of slot ids)
    int count = 0, later_local = 0;
    for (int base = 0; base < S; base += kSlotsPerBlock) {
      int rb[kSlotsPerLane];
      load_roles(r, S, base, lane, rb);
      unsigned kept_bits = 0;
      int loc_after = 0;
#pragma unroll
      for (int j = 0; j < kSlotsPerLane; ++j) {
        int s = base + lane * kSlotsPerLane + j;
        bool la = rb[j] == NATS_ROLE_LOCAL && s > last_g;
        loc_after += la;
        if (s < S_eff && (rb[j] == NATS_ROLE_GLOBAL || la)) kept_bits |= 1u << j;
      }
      int mine = __builtin_popcount(kept_bits);
      int rank = count + wave_excl_scan(mine, lane);
#pragma unroll
      for (int j = 0; j < kSlotsPerLane; ++j) {
        if (kept_bits & (1u << j)) keep[rank++] = base + lane * kSlotsPerLane + j;
      }
      count += wave_sum(mine);
      later_local += wave_sum(loc_after);
    }
    int n_glob = n_glob_all - (partial ? 1 : 0);                                                      // :782-786
    long long n_other = (long long)S - (last_g > 0 ? last_g : 0) - later_local - (partial ? 1 : 0);  // :797-800
    long long dec_l = (last_g > -1 ? (long long)last_g * C + sl : 0) + n_other * C;                  // :793, :802
    hp.count = count;
    hp.dst_base = (int32_t)((last_g == -1 ? sg + sl : sg) / C);                                      // :827-828
    hp.sg_new = sg + (long long)n_glob * C;
    hp.sl_new = sl - dec_l + (long long)n_done * C;
    hp.all_sw = n_sw == S;
    hp.all_local = n_loc == S;
  }
  if (lane == 0) {
    if (kCoherent) {
      // (read by another workgroup of the same launch: written through to where every compute unit reads it)
      const uint64_t* w = reinterpret_cast<const uint64_t*>(&hp);
      uint64_t* dst = reinterpret_cast<uint64_t*>(plans + head);
#pragma unroll
      for (int i = 0; i < (int)(sizeof(HeadPlan) / 8); ++i) __hip_atomic_store(dst + i, w[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
      plans[head] = hp;
    }
  }
}

// The same plan for a head with few role slots, computed by one lane on its own (no wave-wide steps), so that a
// workgroup plans 256 heads side by side.
__device__ __forceinline__ void plan_one_head_serial(const uint8_t* __restrict__ roles, const int64_t* __restrict__ size_global,
                                                     const int64_t* __restrict__ size_local, const nats_evict_params& p,
                                                     char* __restrict__ ws, int head) {
  const int n_heads = (int)(p.B * p.H_kv);
  const int S = (int)p.S;
  const int C = (int)p.C;
  const int partial = (int)(p.fill % p.C);
  const int n_done = (int)(p.fill / p.C);
  const int S_eff = S - (partial ? 1 : 0);
  HeadPlan* plans = reinterpret_cast<HeadPlan*>(ws + kPlanHeaderBytes);
  int32_t* keep = reinterpret_cast<int32_t*>(ws + plan_lists_offset(n_heads)) + (int64_t)head * S;
  const uint8_t* r = roles + (int64_t)head * S;
  const long long sg = old_size_global(p, size_global, head), sl = old_size_local(p, size_local, head);
  HeadPlan hp;
  if (one_step_scatter(p)) {
    int r0 = r[0], rl = r[S - 1];
    bool is_g = r0 == NATS_ROLE_GLOBAL;
    long long dst = is_g ? sg : sg + sl;
    long long dec = (is_g ? sl / C + 1 : 0) + (rl == NATS_ROLE_SW ? 1 : 0);
    hp.count = 1;
    hp.dst_base = (int32_t)(dst / C);
    hp.sg_new = sg + (is_g ? C : 0);
    hp.sl_new = sl - dec * C + (long long)n_done * C;
    hp.all_sw = r0 == NATS_ROLE_SW;
    hp.all_local = 0;
    keep[0] = 0;
  } else {
    int n_glob_all = 0, n_sw = 0, n_loc = 0, last_g = -1;
    for (int s2 = 0; s2 < S; ++s2) {
      const int role = r[s2];
      n_glob_all += role == NATS_ROLE_GLOBAL;
      n_sw += role == NATS_ROLE_SW;
      n_loc += role == NATS_ROLE_LOCAL;
      if (role == NATS_ROLE_GLOBAL && s2 < S_eff) last_g = s2;
    }
    int count = 0, later_local = 0;
    for (int s2 = 0; s2 < S; ++s2) {
      const int role = r[s2];
      const bool la = role == NATS_ROLE_LOCAL && s2 > last_g;
      later_local += la;
      if (s2 < S_eff && (role == NATS_ROLE_GLOBAL || la)) keep[count++] = s2;
    }
    int n_glob = n_glob_all - (partial ? 1 : 0);
    long long n_other = (long long)S - (last_g > 0 ? last_g : 0) - later_local - (partial ? 1 : 0);
    long long dec_l = (last_g > -1 ? (long long)last_g * C + sl : 0) + n_other * C;
    hp.count = count;
    hp.dst_base = (int32_t)((last_g == -1 ? sg + sl : sg) / C);
    hp.sg_new = sg + (long long)n_glob * C;
    hp.sl_new = sl - dec_l + (long long)n_done * C;
    hp.all_sw = n_sw == S;
    hp.all_local = n_loc == S;
  }
  plans[head] = hp;
}

// plan, step 2: one workgroup folds the per-head plans into the global decisions and scalars.
struct PlanAgg {
  int all_sw, all_local;
  int max_keep, max_end;
  long long max_tot_new, max_tot_old, max_tot_alllocal, min_sg_new, min_sg_old, sum_keep;
};

__device__ __forceinline__ void fold(PlanAgg& a, const PlanAgg& b) {
  a.all_sw &= b.all_sw;
  a.all_local &= b.all_local;
  a.max_keep = max(a.max_keep, b.max_keep);
  a.max_end = max(a.max_end, b.max_end);
  a.max_tot_new = max(a.max_tot_new, b.max_tot_new);
  a.max_tot_old = max(a.max_tot_old, b.max_tot_old);
  a.max_tot_alllocal = max(a.max_tot_alllocal, b.max_tot_alllocal);
  a.min_sg_new = min(a.min_sg_new, b.min_sg_new);
  a.min_sg_old = min(a.min_sg_old, b.min_sg_old);
  a.sum_keep += b.sum_keep;
}

static_assert(sizeof(HeadPlan) == 32, "a head plan travels as four 64-bit words");

template <bool kCoherent = false>
__device__ __forceinline__ void plan_finalize(const int64_t* __restrict__ size_global, const int64_t* __restrict__ size_local,
                                              const nats_evict_params& p, char* __restrict__ ws,
                                              nats_evict_result* __restrict__ result,
                                              nats_evict_brief* __restrict__ result_mirror) {
  __shared__ PlanAgg agg[256];
  __shared__ int all_local_flag;
  const int tid = threadIdx.x;
  const int n_heads = (int)(p.B * p.H_kv);
  const int S = (int)p.S;
  const int C = (int)p.C;
  const int partial = (int)(p.fill % p.C);
  const int n_done = (int)(p.fill / p.C);
  HeadPlan* plans = reinterpret_cast<HeadPlan*>(ws + kPlanHeaderBytes);
  PlanAgg w;
  w.all_sw = 1; w.all_local = 1; w.max_keep = 0; w.max_end = 0;
  w.max_tot_new = 0; w.max_tot_old = 0; w.max_tot_alllocal = 0;
  w.min_sg_new = 0x7fffffffffffffffLL; w.min_sg_old = 0x7fffffffffffffffLL; w.sum_keep = 0;
  for (int h = tid; h < n_heads; h += 256) {
    HeadPlan hp;
    if (kCoherent) {  // plans written by other workgroups of this launch
      uint64_t w[sizeof(HeadPlan) / 8];
      const uint64_t* src = reinterpret_cast<const uint64_t*>(plans + h);
#pragma unroll
      for (int i = 0; i < (int)(sizeof(HeadPlan) / 8); ++i) w[i] = __hip_atomic_load(src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      hp = *reinterpret_cast<const HeadPlan*>(w);
    } else {
      hp = plans[h];
    }
    const long long sg = old_size_global(p, size_global, h), sl = old_size_local(p, size_local, h);
    PlanAgg x;
    x.all_sw = hp.all_sw; x.all_local = hp.all_local;
    x.max_keep = hp.count; x.max_end = hp.count + hp.dst_base;
    x.max_tot_new = hp.sg_new + hp.sl_new; x.max_tot_old = sg + sl;
    x.max_tot_alllocal = sg + sl + (long long)n_done * C;
    x.min_sg_new = hp.sg_new; x.min_sg_old = sg; x.sum_keep = hp.count;
    fold(w, x);
  }
  agg[tid] = w;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (tid < o) fold(agg[tid], agg[tid + o]);
    __syncthreads();
  }
  if (tid == 0) {
    const PlanAgg t = agg[0];
    nats_evict_result res;
    res.all_sw = t.all_sw;
    res.all_local = !one_step_scatter(p) && t.all_local && !t.all_sw;
    res.max_keep = t.max_keep;
    res.max_end = t.max_end;
    res.seq = p.seq;
    if (res.all_sw) {  // :283-288; the per-token cache keeps the block where it is (nats_layer_cache.py:316-327)
      res.n_ctx_data = p.update_chunk ? p.n_ctx_data + p.fill : t.max_tot_old + partial;
      res.gmin = p.gmin;
      res.moved_rows = 0;
    } else if (res.all_local) {  // :747-749, then :356-358, :371
      res.n_ctx_data = t.max_tot_alllocal + partial;
      res.gmin = t.min_sg_old;
      res.moved_rows = 0;
    } else {
      res.n_ctx_data = t.max_tot_new + partial;
      res.gmin = t.min_sg_new;
      bool tail_move = !one_step_scatter(p) && partial && t.max_keep < S - 1;  // :840
      res.moved_rows = (t.sum_keep + (tail_move ? n_heads : 0)) * (long long)C;
    }
    *result = res;
    if (result_mirror) {
      // what a host may be polling for (pinned memory): one 16-byte store, so that whoever sees the sequence number
      // sees the rest with it and no fence has to order several stores
      nats_evict_brief m;
      m.seq = (int32_t)p.seq;
      m.flags = (int32_t)(res.all_sw | (res.all_local << 1));
      m.n_ctx_data = (int32_t)res.n_ctx_data;
      m.gmin = (int32_t)res.gmin;
      *reinterpret_cast<uint4*>(result_mirror) = *reinterpret_cast<const uint4*>(&m);
    }
    all_local_flag = (int)res.all_local;
  }
  __syncthreads();
  if (all_local_flag) {
    // every slot local: nothing moves and only the local size grows (:747-749, :356)
    for (int h = tid; h < n_heads; h += 256) {
      plans[h].sg_new = old_size_global(p, size_global, h);
      plans[h].sl_new = old_size_local(p, size_local, h) + (long long)n_done * C;
    }
  }
}

// Few role slots per head (a chunk boundary while decoding or streaming): one workgroup, a lane per head, folds the
// heads itself, so that nothing has to cross workgroups.
__global__ __launch_bounds__(256) void evict_plan_small_kernel(const uint8_t* __restrict__ roles,
                                                               const int64_t* __restrict__ size_global,
                                                               const int64_t* __restrict__ size_local, nats_evict_params p,
                                                               char* __restrict__ ws, nats_evict_result* __restrict__ result,
                                                               nats_evict_brief* __restrict__ result_mirror) {
  const int n_heads = (int)(p.B * p.H_kv);
  for (int head = threadIdx.x; head < n_heads; head += 256) plan_one_head_serial(roles, size_global, size_local, p, ws, head);
  __syncthreads();  // (global writes of this workgroup are visible to it after the barrier)
  plan_finalize(size_global, size_local, p, ws, result, result_mirror);
}

// Many role bytes (a prefill): a wavefront per head over the whole device; the workgroup that draws the launch's last
// ticket (a counter at the start of the workspace, zero between launches) folds the heads.  The per-head plans cross
// from the other workgroups to that one inside the launch, so they are written and read past the caches.
__global__ __launch_bounds__(256) void evict_plan_heads_kernel(const uint8_t* __restrict__ roles,
                                                               const int64_t* __restrict__ size_global,
                                                               const int64_t* __restrict__ size_local, nats_evict_params p,
                                                               char* __restrict__ ws, nats_evict_result* __restrict__ result,
                                                               nats_evict_brief* __restrict__ result_mirror) {
  __shared__ int last;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int head = blockIdx.x * 4 + wave;
  if (head < (int)(p.B * p.H_kv)) plan_one_head<true>(roles, size_global, size_local, p, ws, head, lane);
  __builtin_amdgcn_s_waitcnt(0);  // this workgroup's plans have arrived before it is counted
  __syncthreads();
  if (tid == 0) {
    int32_t* ticket = reinterpret_cast<int32_t*>(ws);
    const int t = atomicAdd(ticket, 1);
    last = t == (int)gridDim.x - 1;
    if (last) atomicExch(ticket, 0);
  }
  __syncthreads();
  if (last) plan_finalize<true>(size_global, size_local, p, ws, result, result_mirror);
}

// ---------------------------------------------------------------------------------------------------
// movers
// ---------------------------------------------------------------------------------------------------
struct ApplyArgs {
  void* tensor[3];       // cache_k, cache_v, pos (pos may be NULL)
  const void* src[2];    // raw K, V of the prefill (out-of-place only)
  uint8_t* valid;
  const uint8_t* roles;
  int64_t* size_global;
  int64_t* size_local;
  const char* ws;
  const nats_evict_result* result;
  nats_evict_params p;
  int64_t ks_b, ks_h, ks_r;  // cache strides in elements
  int64_t ss_b, ss_h, ss_r;  // raw K / V strides in elements (out-of-place only)
  int64_t vs_b, vs_h;        // valid strides; pos uses the same (contiguous rows)
  int elem_bytes;
  int rs;                    // rows per slice
  int n_slices;
  int chunks_per_wg;         // out-of-place only: destination chunks per workgroup
  int64_t n_chunks;          // out-of-place only: destination chunks per head
};

// A tensor seen as units of type U: row `r` of head `head` starts at base + r * row_stride, holds upr units.
template <typename U>
struct TensorView {
  U* base;
  int64_t row_stride;
  int upr;
};

constexpr int kFirstUnr = 4;  // 16-byte units a thread of the out-of-place kernel has in flight
constexpr int kUnr = 4;  // moves per wavefront and batch
constexpr int kNu = 2;   // units per lane and chunk slice (a slice holds at most 128 units)

template <typename U>
__device__ __forceinline__ U zero_unit();
template <>
__device__ __forceinline__ uint4 zero_unit<uint4>() { return make_uint4(0, 0, 0, 0); }
template <>
__device__ __forceinline__ int32_t zero_unit<int32_t>() { return -1; }  // "no token" in the position shadow

template <typename U>
__device__ void apply_inplace_body(const ApplyArgs& a, TensorView<U> t, int head, int slice, bool owns_valid) {
  const nats_evict_params& p = a.p;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int C = (int)p.C, S = (int)p.S;
  const int partial = (int)(p.fill % p.C);
  const int n_done = (int)(p.fill / p.C);
  const int wc = (int)(p.W / p.C);
  const int64_t off = p.n_ctx_data / p.C;
  const int n_heads = (int)(p.B * p.H_kv);
  const nats_evict_result res = *a.result;
  const HeadPlan hp = reinterpret_cast<const HeadPlan*>(a.ws + kPlanHeaderBytes)[head];
  const int32_t* keep = reinterpret_cast<const int32_t*>(a.ws + plan_lists_offset(n_heads)) + (int64_t)head * S;
  const uint8_t* r = a.roles + (int64_t)head * S;
  const int units = a.rs * t.upr;  // per chunk slice
  const int row0 = slice * a.rs;

  auto unit_ptr = [&](int64_t chunk, int u) -> U* {
    return t.base + (chunk * C + row0 + u / t.upr) * t.row_stride + (u % t.upr);
  };

  // 1. ring insert (:391-437)
  const bool token = p.update_chunk != 0;
  const int n_ring = n_done < wc ? n_done : wc;
  // the chunked cache's tail is the next slot to write, the per-token cache's the slot written last; its one-step
  // branch writes one slot further on (nats_layer_cache.py:340-345: slot 1 for the first token ever, else tail + 2,
  // while the tail itself advances by one), unless every head's token is sliding-window (:316-317)
  const int skip = token && one_step_scatter(p) && !res.all_sw ? 1 : 0;
  const int start_chunk = p.first ? skip : token ? (int)((p.tail + 1 + skip) % p.W) : (int)(p.tail / p.C);
  for (int j = wave; j < n_ring; j += 4) {
    int slot = n_done - n_ring + j;
    bool is_sw = r[slot] == NATS_ROLE_SW;
    int rc = (start_chunk + j) % wc;
    for (int u = lane; u < units; u += kWave) {
      U val = (is_sw || token) ? *unit_ptr(off + slot, u) : zero_unit<U>();  // (nats_layer_cache.py:451-454 copies all)
      *unit_ptr(rc, u) = val;
    }
    if (owns_valid && lane < a.rs) {
      a.valid[(int64_t)(head / p.H_kv) * a.vs_b + (int64_t)(head % p.H_kv) * a.vs_h + (int64_t)rc * C + row0 + lane] = is_sw;
    }
  }
  if (res.all_sw) return;
  __syncthreads();

  // 2. ordered chunk moves, each batch read completely before it is written
  int n_moves;
  bool tail_move = false;
  if (one_step_scatter(p)) {
    n_moves = 1;
  } else if (res.all_local) {
    n_moves = 0;
  } else {
    tail_move = partial && res.max_keep < S - 1;
    n_moves = hp.count + (tail_move ? 1 : 0);
  }
  for (int b0 = 0; b0 < n_moves; b0 += 4 * kUnr) {
    U regs[kUnr][kNu];
    int64_t dsts[kUnr];
#pragma unroll
    for (int k = 0; k < kUnr; ++k) {
      int mv = b0 + wave * kUnr + k;
      dsts[k] = -1;
      if (mv < n_moves) {
        int64_t src, dst;
        if (mv < hp.count) {
          src = off + keep[mv];
          dst = hp.dst_base + mv;
        } else {
          src = off + S - 1;
          dst = res.max_end;
        }
        if (src != dst) {
          dsts[k] = dst;
#pragma unroll
          for (int e = 0; e < kNu; ++e) {
            int u = lane + e * kWave;
            if (u < units) regs[k][e] = *unit_ptr(src, u);
          }
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kUnr; ++k) {
      if (dsts[k] >= 0) {
#pragma unroll
        for (int e = 0; e < kNu; ++e) {
          int u = lane + e * kWave;
          if (u < units) *unit_ptr(dsts[k], u) = regs[k][e];
        }
      }
    }
  }
  __syncthreads();

  // 3. rows >= n_ctx_data are zeroed (:360-362); the per-token cache leaves them as they are
  const int64_t n_chunks_alloc = token ? 0 : p.n_alloc / C;
  for (int64_t ci = res.n_ctx_data / C + wave; ci < n_chunks_alloc; ci += 4) {
    for (int u = lane; u < units; u += kWave) {
      int64_t row = ci * C + row0 + u / t.upr;
      if (row >= res.n_ctx_data) *unit_ptr(ci, u) = zero_unit<U>();
    }
  }

  if (owns_valid) {
    // 4. valid_tokens rewrite with the minimum global size from before this call (:634-656)
    const long long sg_new = hp.sg_new, sl_new = hp.sl_new;
    if (res.n_ctx_data != p.gmin) {
      uint8_t* vrow = a.valid + (int64_t)(head / p.H_kv) * a.vs_b + (int64_t)(head % p.H_kv) * a.vs_h;
      const int64_t last_chunk = res.n_ctx_data / C * C;
      const int64_t hi = last_chunk + partial;
      for (int64_t i = p.gmin + slice * 256 + tid; i < hi; i += (int64_t)a.n_slices * 256) {
        vrow[i] = i < last_chunk ? (i < sg_new + sl_new) : 1;
      }
    }
    if (slice == 0 && tid == 0) {
      a.size_global[head] = sg_new;
      a.size_local[head] = sl_new;
    }
  }
}

__global__ __launch_bounds__(256) void evict_apply_inplace_kernel(ApplyArgs a) {
  const int slice = blockIdx.x;
  const int head = blockIdx.y;
  const int which = blockIdx.z;
  const int b = head / (int)a.p.H_kv, h = head % (int)a.p.H_kv;
  if (which < 2) {
    TensorView<uint4> t;
    int row_units = (int)(a.p.D * a.elem_bytes / 16);
    t.base = reinterpret_cast<uint4*>(static_cast<char*>(a.tensor[which]) + (b * a.ks_b + h * a.ks_h) * a.elem_bytes);
    t.row_stride = a.ks_r * a.elem_bytes / 16;
    t.upr = row_units;
    apply_inplace_body<uint4>(a, t, head, slice, which == 0);
  } else {
    TensorView<int32_t> t;
    t.base = static_cast<int32_t*>(a.tensor[2]) + b * a.vs_b + h * a.vs_h;
    t.row_stride = 1;
    t.upr = 1;
    apply_inplace_body<int32_t>(a, t, head, slice, false);
  }
}

// Out of place, first prefill: destination chunks [blockIdx.x * chunks_per_wg, +chunks_per_wg) of head blockIdx.y
// (several chunks per workgroup when a chunk is shorter than 32 rows, so that a workgroup moves 16 KiB).
__global__ __launch_bounds__(256) void evict_apply_first_kernel(ApplyArgs a) {
  const nats_evict_params& p = a.p;
  const int tid = threadIdx.x;
  const int head = blockIdx.y;
  const int which = blockIdx.z;
  const int b = head / (int)p.H_kv, h = head % (int)p.H_kv;
  const int C = (int)p.C, S = (int)p.S;
  const int partial = (int)(p.fill % p.C);
  const int n_done = (int)(p.fill / p.C);
  const int wc = (int)(p.W / p.C);
  const int64_t L = p.x_len;
  const int n_heads = (int)(p.B * p.H_kv);
  const nats_evict_result res = *a.result;
  if (res.all_sw) return;  // the reference leaves the untruncated cache in this case; not handled out of place
  const HeadPlan hp = reinterpret_cast<const HeadPlan*>(a.ws + kPlanHeaderBytes)[head];
  const int32_t* keep = reinterpret_cast<const int32_t*>(a.ws + plan_lists_offset(n_heads)) + (int64_t)head * S;
  const uint8_t* r = a.roles + (int64_t)head * S;
  const int n_ring = n_done < wc ? n_done : wc;
  const int count = res.all_local ? 0 : hp.count;
  const bool tail_move = !res.all_local && partial && res.max_keep < S - 1;

  // Destination chunks past the last one that holds live rows are spare capacity (a cache allocated on a guess of
  // its size): they are left as they are; whoever extends the cache into them initialises them then.
  const int64_t ci_end = min(min((int64_t)(blockIdx.x + 1) * a.chunks_per_wg, a.n_chunks), (res.n_ctx_data + C - 1) / C);
  for (int64_t ci = (int64_t)blockIdx.x * a.chunks_per_wg; ci < ci_end; ++ci) {
  // where the rows of this destination chunk come from: a source chunk of the raw prefill tensor
  // (-1 = zeros); the untouched part of [W zeros | K | pad] keeps its own rows
  int64_t src_chunk;
  bool ring_sw = false;  // a ring chunk whose tokens are sliding-window (valid)
  if (ci < wc) {
    src_chunk = -1;
    if (ci < n_ring) {
      int slot = n_done - n_ring + (int)ci;
      ring_sw = r[slot] == NATS_ROLE_SW;
      if (ring_sw || p.update_chunk) src_chunk = slot;  // the per-token cache copies the row whatever the role
    }
  } else {
    int64_t rel = ci - hp.dst_base;
    if (rel >= 0 && rel < count) {
      src_chunk = keep[rel];
    } else if (tail_move && ci == res.max_end) {
      src_chunk = S - 1;
    } else {
      src_chunk = ci - wc;
    }
  }

  const long long sg_new = hp.sg_new, sl_new = hp.sl_new;

  if (which < 2) {
    const int upr = (int)(p.D * a.elem_bytes / 16);
    uint4* dst = reinterpret_cast<uint4*>(static_cast<char*>(a.tensor[which]) + (b * a.ks_b + h * a.ks_h) * a.elem_bytes);
    const uint4* src =
        reinterpret_cast<const uint4*>(static_cast<const char*>(a.src[which]) + (b * a.ss_b + h * a.ss_h) * a.elem_bytes);
    const int64_t d_stride = a.ks_r * a.elem_bytes / 16, s_stride = a.ss_r * a.elem_bytes / 16;
    // Every row is read once and written once: both sides carry the streaming hint.  A thread has kFirstUnr loads
    // in flight before its first store (a 64-row chunk of 256-byte rows is one trip).
    const int n_units = C * upr;
    const int row_step = 256 / upr, col_step = 256 % upr;
    int row = tid / upr, col = tid % upr;
    for (int u0 = tid; u0 < n_units; u0 += 256 * kFirstUnr) {
      u32x4 val[kFirstUnr];
      uint4* to[kFirstUnr];
#pragma unroll
      for (int k = 0; k < kFirstUnr; ++k) {
        val[k] = u32x4{0u, 0u, 0u, 0u};
        to[k] = nullptr;
        if (u0 + k * 256 < n_units) {
          const int64_t drow = ci * C + row;
          const int64_t tok = src_chunk < 0 ? -1 : src_chunk * C + row;
          to[k] = dst + drow * d_stride + col;
          if (tok >= 0 && tok < L && drow < res.n_ctx_data) {
            val[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + tok * s_stride + col));
          }
        }
        row += row_step;
        col += col_step;
        if (col >= upr) {
          col -= upr;
          ++row;
        }
      }
#pragma unroll
      for (int k = 0; k < kFirstUnr; ++k) {
        if (to[k]) __builtin_nontemporal_store(val[k], reinterpret_cast<u32x4*>(to[k]));
      }
    }
  } else {
    int32_t* dst = static_cast<int32_t*>(a.tensor[2]) + b * a.vs_b + h * a.vs_h;
    for (int row = tid; row < C; row += 256) {
      int64_t drow = ci * C + row;
      int64_t tok = src_chunk < 0 ? -1 : src_chunk * C + row;
      dst[drow] = (tok >= 0 && tok < L && drow < res.n_ctx_data) ? (int32_t)tok : -1;
    }
  }

  if (which == 0) {
    uint8_t* vrow = a.valid + (int64_t)b * a.vs_b + (int64_t)h * a.vs_h;
    const int64_t last_chunk = res.n_ctx_data / C * C;
    for (int row = tid; row < C; row += 256) {
      int64_t i = ci * C + row;
      uint8_t v;
      if (i < p.W) {
        v = ring_sw ? 1 : 0;
      } else {
        v = (i - p.W) < L ? 1 : 0;  // what update() left behind (:229-236)
        if (res.n_ctx_data != p.gmin && i >= p.gmin) {
          if (i < last_chunk) {
            v = i < sg_new + sl_new;
          } else if (i < last_chunk + partial) {
            v = 1;
          }
        }
      }
      vrow[i] = v;
    }
    if (ci == 0 && tid == 0) {
      a.size_global[head] = sg_new;
      a.size_local[head] = sl_new;
    }
  }
  }  // chunks of this workgroup
}

// Rows of new keys / values into the cache, 16 bytes per lane, with their valid bytes and stream positions.
struct AppendArgs {
  const void* src[2];
  void* dst[2];
  uint8_t* valid;
  int32_t* pos;
  int64_t ss[2][3];  // strides (b, h, l) of k and of v, in 16-byte units
  int64_t ds[3];     // cache strides (b, h, row), in 16-byte units
  int64_t vs_b, vs_h;
  int64_t row0, pos0;
  int x_len, upr, H_kv;
};

__global__ __launch_bounds__(256) void cache_append_kernel(AppendArgs a) {
  const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int head = blockIdx.y, which = blockIdx.z;
  const int b = head / a.H_kv, h = head % a.H_kv;
  const int64_t l = u / a.upr;
  const int col = (int)(u % a.upr);
  if (l >= a.x_len) return;
  const uint4* src = static_cast<const uint4*>(a.src[which]) + b * a.ss[which][0] + h * a.ss[which][1] + l * a.ss[which][2] + col;
  uint4* dst = static_cast<uint4*>(a.dst[which]) + b * a.ds[0] + h * a.ds[1] + (a.row0 + l) * a.ds[2] + col;
  *dst = *src;
  if (which == 0 && col == 0) {
    const int64_t at = b * a.vs_b + h * a.vs_h + a.row0 + l;
    a.valid[at] = 1;
    if (a.pos) a.pos[at] = (int32_t)(a.pos0 + l);
  }
}

// The append and the plan of the eviction that follows it in one launch: the last workgroup along x (of head 0,
// tensor 0) has no rows to copy and runs the small plan kernel's work instead.  What the plan reads (roles, sizes,
// the host's scalars) does not depend on the rows being appended.
__global__ __launch_bounds__(256) void cache_append_plan_kernel(AppendArgs a, const uint8_t* __restrict__ roles,
                                                                const int64_t* __restrict__ size_global,
                                                                const int64_t* __restrict__ size_local, nats_evict_params p,
                                                                char* __restrict__ ws, nats_evict_result* __restrict__ result,
                                                                nats_evict_brief* __restrict__ result_mirror) {
  if (blockIdx.x + 1 < gridDim.x) {
    const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int head = blockIdx.y, which = blockIdx.z;
    const int b = head / a.H_kv, h = head % a.H_kv;
    const int64_t l = u / a.upr;
    const int col = (int)(u % a.upr);
    if (l >= a.x_len) return;
    const uint4* src = static_cast<const uint4*>(a.src[which]) + b * a.ss[which][0] + h * a.ss[which][1] + l * a.ss[which][2] + col;
    uint4* dst = static_cast<uint4*>(a.dst[which]) + b * a.ds[0] + h * a.ds[1] + (a.row0 + l) * a.ds[2] + col;
    *dst = *src;
    if (which == 0 && col == 0) {
      const int64_t at = b * a.vs_b + h * a.vs_h + a.row0 + l;
      a.valid[at] = 1;
      if (a.pos) a.pos[at] = (int32_t)(a.pos0 + l);
    }
    return;
  }
  if (blockIdx.y != 0 || blockIdx.z != 0) return;
  const int n_heads = (int)(p.B * p.H_kv);
  for (int head = threadIdx.x; head < n_heads; head += 256) plan_one_head_serial(roles, size_global, size_local, p, ws, head);
  __syncthreads();  // (global writes of this workgroup are visible to it after the barrier)
  plan_finalize(size_global, size_local, p, ws, result, result_mirror);
}

static int check_params(const char* who, const nats_evict_params* p) {
  NATS_REQUIRE(p, NATS_ERR_NULL_POINTER, "%s: params must not be NULL", who);
  NATS_REQUIRE(p->B > 0 && p->H_kv > 0 && p->D > 0 && p->S > 0, NATS_ERR_BAD_SHAPE, "%s: B=%lld H_kv=%lld D=%lld S=%lld", who,
               (long long)p->B, (long long)p->H_kv, (long long)p->D, (long long)p->S);
  NATS_REQUIRE(p->C > 0 && p->W > 0 && p->W % p->C == 0, NATS_ERR_BAD_SHAPE,
               "%s: window %lld is not a positive multiple of chunk size %lld", who, (long long)p->W, (long long)p->C);
  NATS_REQUIRE(p->x_len > 0 && p->fill >= p->C && p->fill >= p->x_len, NATS_ERR_BAD_SHAPE,
               "%s: x_len=%lld fill=%lld: no chunk completed, nothing to evict", who, (long long)p->x_len, (long long)p->fill);
  int64_t n_done = p->fill / p->C, partial = p->fill % p->C;
  NATS_REQUIRE(p->S == n_done + (partial ? 1 : 0), NATS_ERR_BAD_SHAPE, "%s: S=%lld role slots for fill=%lld, chunk %lld", who,
               (long long)p->S, (long long)p->fill, (long long)p->C);
  NATS_REQUIRE(p->update_chunk >= 0 && (p->update_chunk == 0 || (p->C == 1 && p->fill >= p->update_chunk && p->update_chunk <= p->W)),
               NATS_ERR_BAD_SHAPE, "%s: update_chunk=%lld needs chunk size 1, a window and a pending block of at least that many tokens",
               who, (long long)p->update_chunk);
  NATS_REQUIRE(p->x_len != 1 || p->S == 1 || p->update_chunk > 1, NATS_ERR_BAD_SHAPE, "%s: a one-token step completes exactly one chunk", who);
  NATS_REQUIRE(p->update_chunk != 1 || p->W >= 2, NATS_ERR_UNSUPPORTED, "%s: update_chunk=1 needs a window of at least two tokens", who);
  NATS_REQUIRE(p->n_ctx_data >= p->W && p->gmin >= p->W && p->tail >= 0 && p->tail < p->W && p->tail % p->C == 0,
               NATS_ERR_BAD_SHAPE, "%s: n_ctx_data=%lld gmin=%lld tail=%lld", who, (long long)p->n_ctx_data,
               (long long)p->gmin, (long long)p->tail);
  NATS_REQUIRE(p->B * p->H_kv <= 65535, NATS_ERR_BAD_SHAPE, "%s: too many (b, head) streams", who);
  return NATS_OK;
}

}  // namespace nats

using namespace nats;

extern "C" size_t nats_evict_workspace_bytes(int64_t B, int64_t H_kv, int64_t S) {
  if (B <= 0 || H_kv <= 0 || S <= 0) return 0;
  return plan_lists_offset(B * H_kv) + (size_t)(B * H_kv * S) * sizeof(int32_t);
}

extern "C" int nats_evict_plan(const uint8_t* roles, const int64_t* size_global, const int64_t* size_local,
                               const nats_evict_params* params, void* workspace, size_t workspace_bytes,
                               nats_evict_result* result, nats_evict_brief* result_mirror, void* stream) {
  NATS_REQUIRE(roles && size_global && size_local && workspace && result, NATS_ERR_NULL_POINTER,
               "nats_evict_plan: NULL pointer argument");
  if (int rc = check_params("nats_evict_plan", params)) return rc;
  size_t need = nats_evict_workspace_bytes(params->B, params->H_kv, params->S);
  NATS_REQUIRE(workspace_bytes >= need, NATS_ERR_WORKSPACE, "nats_evict_plan: workspace %zu bytes < %zu", workspace_bytes, need);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const unsigned n_wg = (unsigned)((params->B * params->H_kv + 3) / 4);
  if (params->S <= 32 && params->B * params->H_kv <= 4096) {
    hipLaunchKernelGGL(evict_plan_small_kernel, dim3(1), dim3(256), 0, st, roles, size_global, size_local, *params,
                       static_cast<char*>(workspace), result, result_mirror);
    NATS_CHECK_LAUNCH("evict_plan_small_kernel");
    return NATS_OK;
  }
  hipLaunchKernelGGL(evict_plan_heads_kernel, dim3(n_wg), dim3(256), 0, st, roles, size_global, size_local, *params,
                     static_cast<char*>(workspace), result, result_mirror);
  NATS_CHECK_LAUNCH("evict_plan_heads_kernel");
  return NATS_OK;
}

static int slice_geometry(const char* who, const nats_evict_params* p, int elem_bytes, int* rs, int* n_slices) {
  NATS_REQUIRE(elem_bytes == 2 || elem_bytes == 4, NATS_ERR_BAD_DTYPE, "%s: element size %d", who, elem_bytes);
  int64_t row_bytes = p->D * elem_bytes;
  NATS_REQUIRE(row_bytes % 16 == 0 && row_bytes <= 2048, NATS_ERR_UNSUPPORTED, "%s: row of %lld bytes", who,
               (long long)row_bytes);
  int64_t r = 1;
  while (r * 2 <= p->C && r * 2 * row_bytes <= 2048 && p->C % (r * 2) == 0) r *= 2;
  NATS_REQUIRE(p->C % r == 0, NATS_ERR_UNSUPPORTED, "%s: chunk size %lld", who, (long long)p->C);
  if (r > 128) r = 128;  // the position shadow moves one 4-byte unit per row
  *rs = (int)r;
  *n_slices = (int)(p->C / r);
  return NATS_OK;
}

extern "C" int nats_evict_apply_inplace(void* cache_k, void* cache_v, uint8_t* valid, int32_t* pos, const uint8_t* roles,
                                        int64_t* size_global, int64_t* size_local, const nats_evict_params* params,
                                        const int64_t* kv_strides, const int64_t* valid_strides, int elem_bytes,
                                        const void* workspace, const nats_evict_result* result, void* stream) {
  NATS_REQUIRE(cache_k && cache_v && valid && roles && size_global && size_local && workspace && result,
               NATS_ERR_NULL_POINTER, "nats_evict_apply_inplace: NULL pointer argument");
  NATS_REQUIRE(kv_strides && valid_strides, NATS_ERR_NULL_POINTER, "nats_evict_apply_inplace: NULL stride array");
  if (int rc = check_params("nats_evict_apply_inplace", params)) return rc;
  // rows up to the end of the open-chunk region (the per-token cache hands over the first row of its pending block)
  const int64_t region0 = params->update_chunk ? params->n_ctx_data : params->n_ctx_data - (params->fill - params->x_len);
  NATS_REQUIRE(params->n_alloc % params->C == 0 && params->n_alloc >= region0 + params->fill, NATS_ERR_BAD_SHAPE,
               "nats_evict_apply_inplace: n_alloc=%lld", (long long)params->n_alloc);
  ApplyArgs a;
  if (int rc = slice_geometry("nats_evict_apply_inplace", params, elem_bytes, &a.rs, &a.n_slices)) return rc;
  NATS_REQUIRE((kv_strides[0] * elem_bytes) % 16 == 0 && (kv_strides[1] * elem_bytes) % 16 == 0 &&
                   (kv_strides[2] * elem_bytes) % 16 == 0 &&
                   (reinterpret_cast<uintptr_t>(cache_k) | reinterpret_cast<uintptr_t>(cache_v)) % 16 == 0,
               NATS_ERR_BAD_SHAPE, "nats_evict_apply_inplace: cache rows must be 16-byte aligned");
  a.tensor[0] = cache_k; a.tensor[1] = cache_v; a.tensor[2] = pos;
  a.src[0] = a.src[1] = nullptr;
  a.valid = valid; a.roles = roles; a.size_global = size_global; a.size_local = size_local;
  a.ws = static_cast<const char*>(workspace); a.result = result; a.p = *params;
  a.ks_b = kv_strides[0]; a.ks_h = kv_strides[1]; a.ks_r = kv_strides[2];
  a.ss_b = a.ss_h = a.ss_r = 0;
  a.vs_b = valid_strides[0]; a.vs_h = valid_strides[1];
  a.elem_bytes = elem_bytes;
  dim3 grid((unsigned)a.n_slices, (unsigned)(params->B * params->H_kv), pos ? 3u : 2u);
  hipLaunchKernelGGL(evict_apply_inplace_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), a);
  NATS_CHECK_LAUNCH("evict_apply_inplace_kernel");
  return NATS_OK;
}

extern "C" int nats_evict_apply_first(const void* src_k, const void* src_v, void* cache_k, void* cache_v, uint8_t* valid,
                                      int32_t* pos, const uint8_t* roles, int64_t* size_global, int64_t* size_local,
                                      const nats_evict_params* params, const int64_t* src_strides, const int64_t* kv_strides,
                                      const int64_t* valid_strides, int elem_bytes, const void* workspace,
                                      const nats_evict_result* result, void* stream) {
  NATS_REQUIRE(src_k && src_v && cache_k && cache_v && valid && roles && size_global && size_local && workspace && result,
               NATS_ERR_NULL_POINTER, "nats_evict_apply_first: NULL pointer argument");
  NATS_REQUIRE(src_strides && kv_strides && valid_strides, NATS_ERR_NULL_POINTER, "nats_evict_apply_first: NULL stride array");
  if (int rc = check_params("nats_evict_apply_first", params)) return rc;
  NATS_REQUIRE(params->first == 1 && params->x_len > 1 && params->fill == params->x_len && params->n_ctx_data == params->W &&
                   params->gmin == params->W,
               NATS_ERR_BAD_SHAPE, "nats_evict_apply_first: only the first update of an empty cache can be applied out of place");
  NATS_REQUIRE(params->n_alloc % params->C == 0 && params->n_alloc > 0 && params->n_alloc / params->C <= 0x7fffffff,
               NATS_ERR_BAD_SHAPE, "nats_evict_apply_first: n_alloc=%lld", (long long)params->n_alloc);
  NATS_REQUIRE(elem_bytes == 2 || elem_bytes == 4, NATS_ERR_BAD_DTYPE, "nats_evict_apply_first: element size %d", elem_bytes);
  NATS_REQUIRE((params->D * elem_bytes) % 16 == 0, NATS_ERR_UNSUPPORTED, "nats_evict_apply_first: row of %lld bytes",
               (long long)(params->D * elem_bytes));
  for (int i = 0; i < 3; ++i) {
    NATS_REQUIRE((src_strides[i] * elem_bytes) % 16 == 0 && (kv_strides[i] * elem_bytes) % 16 == 0, NATS_ERR_BAD_SHAPE,
                 "nats_evict_apply_first: rows must be 16-byte aligned");
  }
  NATS_REQUIRE((reinterpret_cast<uintptr_t>(cache_k) | reinterpret_cast<uintptr_t>(cache_v) |
                reinterpret_cast<uintptr_t>(src_k) | reinterpret_cast<uintptr_t>(src_v)) % 16 == 0,
               NATS_ERR_BAD_SHAPE, "nats_evict_apply_first: tensors must be 16-byte aligned");
  ApplyArgs a;
  a.tensor[0] = cache_k; a.tensor[1] = cache_v; a.tensor[2] = pos;
  a.src[0] = src_k; a.src[1] = src_v;
  a.valid = valid; a.roles = roles; a.size_global = size_global; a.size_local = size_local;
  a.ws = static_cast<const char*>(workspace); a.result = result; a.p = *params;
  a.ks_b = kv_strides[0]; a.ks_h = kv_strides[1]; a.ks_r = kv_strides[2];
  a.ss_b = src_strides[0]; a.ss_h = src_strides[1]; a.ss_r = src_strides[2];
  a.vs_b = valid_strides[0]; a.vs_h = valid_strides[1];
  a.elem_bytes = elem_bytes; a.rs = 0; a.n_slices = 0;
  a.n_chunks = params->n_alloc / params->C;
  a.chunks_per_wg = params->C >= 32 ? 1 : (int)(64 / params->C);
  dim3 grid((unsigned)((a.n_chunks + a.chunks_per_wg - 1) / a.chunks_per_wg), (unsigned)(params->B * params->H_kv), pos ? 3u : 2u);
  hipLaunchKernelGGL(evict_apply_first_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), a);
  NATS_CHECK_LAUNCH("evict_apply_first_kernel");
  return NATS_OK;
}

static int fill_append_args(const char* who, AppendArgs& a, const void* k, const void* v, void* cache_k, void* cache_v,
                            uint8_t* valid, int32_t* pos, int64_t B, int64_t H_kv, int64_t x_len, int64_t D, int64_t row0,
                            int64_t n_alloc, int64_t pos0, const int64_t* k_strides, const int64_t* v_strides,
                            const int64_t* cache_strides, const int64_t* valid_strides, int elem_bytes, dim3* grid) {
  NATS_REQUIRE(k && v && cache_k && cache_v && valid, NATS_ERR_NULL_POINTER, "%s: NULL pointer argument", who);
  NATS_REQUIRE(k_strides && v_strides && cache_strides && valid_strides, NATS_ERR_NULL_POINTER, "%s: NULL stride array", who);
  NATS_REQUIRE(B > 0 && H_kv > 0 && x_len > 0 && D > 0 && B * H_kv <= 65535, NATS_ERR_BAD_SHAPE,
               "%s: B=%lld H_kv=%lld x_len=%lld D=%lld", who, (long long)B, (long long)H_kv, (long long)x_len, (long long)D);
  NATS_REQUIRE(row0 >= 0 && row0 + x_len <= n_alloc, NATS_ERR_BAD_SHAPE, "%s: rows [%lld, %lld) of %lld", who,
               (long long)row0, (long long)(row0 + x_len), (long long)n_alloc);
  NATS_REQUIRE(elem_bytes == 2 || elem_bytes == 4, NATS_ERR_BAD_DTYPE, "%s: element size %d", who, elem_bytes);
  NATS_REQUIRE((D * elem_bytes) % 16 == 0, NATS_ERR_UNSUPPORTED, "%s: row of %lld bytes", who, (long long)(D * elem_bytes));
  for (int i = 0; i < 3; ++i) {
    NATS_REQUIRE((k_strides[i] * elem_bytes) % 16 == 0 && (v_strides[i] * elem_bytes) % 16 == 0 &&
                     (cache_strides[i] * elem_bytes) % 16 == 0,
                 NATS_ERR_BAD_SHAPE, "%s: rows must be 16-byte aligned", who);
    a.ss[0][i] = k_strides[i] * elem_bytes / 16;
    a.ss[1][i] = v_strides[i] * elem_bytes / 16;
    a.ds[i] = cache_strides[i] * elem_bytes / 16;
  }
  NATS_REQUIRE((reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) | reinterpret_cast<uintptr_t>(cache_k) |
                reinterpret_cast<uintptr_t>(cache_v)) % 16 == 0,
               NATS_ERR_BAD_SHAPE, "%s: tensors must be 16-byte aligned", who);
  a.src[0] = k; a.src[1] = v; a.dst[0] = cache_k; a.dst[1] = cache_v;
  a.valid = valid; a.pos = pos;
  a.vs_b = valid_strides[0]; a.vs_h = valid_strides[1];
  a.row0 = row0; a.pos0 = pos0;
  a.x_len = (int)x_len; a.upr = (int)(D * elem_bytes / 16); a.H_kv = (int)H_kv;
  const int64_t units = x_len * a.upr;
  NATS_REQUIRE(units < (int64_t(1) << 38), NATS_ERR_BAD_SHAPE, "%s: too many rows", who);
  *grid = dim3((unsigned)((units + 255) / 256), (unsigned)(B * H_kv), 2u);
  return NATS_OK;
}

extern "C" int nats_cache_append(const void* k, const void* v, void* cache_k, void* cache_v, uint8_t* valid, int32_t* pos,
                                 int64_t B, int64_t H_kv, int64_t x_len, int64_t D, int64_t row0, int64_t n_alloc, int64_t pos0,
                                 const int64_t* k_strides, const int64_t* v_strides, const int64_t* cache_strides,
                                 const int64_t* valid_strides, int elem_bytes, void* stream) {
  AppendArgs a;
  dim3 grid;
  if (int rc = fill_append_args("nats_cache_append", a, k, v, cache_k, cache_v, valid, pos, B, H_kv, x_len, D, row0, n_alloc,
                                pos0, k_strides, v_strides, cache_strides, valid_strides, elem_bytes, &grid))
    return rc;
  hipLaunchKernelGGL(cache_append_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), a);
  NATS_CHECK_LAUNCH("cache_append_kernel");
  return NATS_OK;
}

extern "C" int nats_cache_append_plan(const void* k, const void* v, void* cache_k, void* cache_v, uint8_t* valid, int32_t* pos,
                                      int64_t B, int64_t H_kv, int64_t x_len, int64_t D, int64_t row0, int64_t n_alloc,
                                      int64_t pos0, const int64_t* k_strides, const int64_t* v_strides,
                                      const int64_t* cache_strides, const int64_t* valid_strides, int elem_bytes,
                                      const uint8_t* roles, const int64_t* size_global, const int64_t* size_local,
                                      const nats_evict_params* params, void* workspace, size_t workspace_bytes,
                                      nats_evict_result* result, nats_evict_brief* result_mirror, void* stream) {
  const char* who = "nats_cache_append_plan";
  AppendArgs a;
  dim3 grid;
  if (int rc = fill_append_args(who, a, k, v, cache_k, cache_v, valid, pos, B, H_kv, x_len, D, row0, n_alloc, pos0, k_strides,
                                v_strides, cache_strides, valid_strides, elem_bytes, &grid))
    return rc;
  NATS_REQUIRE(roles && size_global && size_local && workspace && result, NATS_ERR_NULL_POINTER, "%s: NULL pointer argument", who);
  if (int rc = check_params(who, params)) return rc;
  NATS_REQUIRE(params->B == B && params->H_kv == H_kv && params->x_len == x_len, NATS_ERR_BAD_SHAPE,
               "%s: the eviction parameters describe another update (B=%lld H_kv=%lld x_len=%lld)", who, (long long)params->B,
               (long long)params->H_kv, (long long)params->x_len);
  NATS_REQUIRE(params->S <= 32 && B * H_kv <= 4096, NATS_ERR_UNSUPPORTED,
               "%s: %lld role slots for %lld heads: the plan that rides with an append takes at most 32 for 4096 (use "
               "nats_cache_append and nats_evict_plan)",
               who, (long long)params->S, (long long)(B * H_kv));
  size_t need = nats_evict_workspace_bytes(params->B, params->H_kv, params->S);
  NATS_REQUIRE(workspace_bytes >= need, NATS_ERR_WORKSPACE, "%s: workspace %zu bytes < %zu", who, workspace_bytes, need);
  grid.x += 1;  // the workgroup that plans
  hipLaunchKernelGGL(cache_append_plan_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), a, roles, size_global,
                     size_local, *params, static_cast<char*>(workspace), result, result_mirror);
  NATS_CHECK_LAUNCH("cache_append_plan_kernel");
  return NATS_OK;
}
