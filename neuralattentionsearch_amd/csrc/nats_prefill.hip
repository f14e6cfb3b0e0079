// Role-masked, chunked flash-attention prefill for gfx950.
//
// Kernels (they share the per-row limits and the tile / granule summaries of the key-limit stage):
//   prefill_mfma_kernel        bf16, QK^T and PV on v_mfma_f32_32x32x16_bf16, fp32 online softmax; walks whole 64-row
//                              key tiles (kMode 0), tiles assembled from the visible 16-row granules (kMode 1), or, for
//                              chunks shorter than a granule, tiles gathered row by row from the lists of long-lived
//                              rows far behind a query plus granules near it (kMode 2); with n_split > 1 several
//                              workgroups share one tile list and leave partial results
//   prefill_split_merge_kernel combines those partial results
//   prefill_mfma_wide_kernel   bf16 MFMA kernel for head dim 256: four wavefronts with the whole register file, whole
//                              tiles masked row by row
//   prefill_simple_kernel      fp32 (or bf16) FMA kernel, one query row per lane; the fp32 parity path
//
// Mask semantics (components/masks/utils.py:89-94, components/cache/nats_chunk_layer_cache.py:462-511, 603-616):
// the queries are tokens [r_begin, r_end) of the open-chunk region, which starts at key row `base`; every key
// row carries the last region token that sees it (tok_lim, built from the roles of the segment and, for
// rows below base, from the state earlier segments left in the cache).  Query token r sees key row n iff
//   r <= tok_lim[n]  and  n - base <= r          (rows below base are older than every query).
// A prefill from an empty cache is the case base = 0, r_begin = 0.
#include <stdlib.h>

#include "nats_common.h"

namespace nats {

struct PrefillArgs {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  const int32_t* tok_lim;  // [B*Hkv, N], then one entry holding -1
  const int2* tile_lim;    // [B*Hkv, Tk] {max, min}
  const int2* gran_lim;    // [B*Hkv, Tk * 4] {max, min} of every 16 key rows
  int64_t qs_b, qs_h, qs_l;
  int64_t ks_b, ks_h, ks_l;
  int64_t vs_b, vs_h, vs_l;
  int64_t os_b, os_h, os_l;
  int B, Hq, Hkv, n_rep;
  int N, Tk;             // key rows and 64-row key tiles
  int base;              // first key row of the region
  int r_begin, r_end;    // region tokens that are queries; query i of q / o is token r_begin + i
  int qt_first, qt_last; // 64-token region tiles that hold queries
  int hpw;       // q heads of one kv head handled by one workgroup (mfma kernel)
  int qpw;       // 64-row query tiles handled by one workgroup (mfma kernel)
  int n_hg;      // head groups per kv head = n_rep / hpw
  int n_qg;      // query tile groups = ceil(n query tiles / qpw)
  int xcd_mode;  // 1: workgroups of one kv stream share an XCD (needs B*Hkv % 8 == 0)
  // The query groups with the fewest visible keys (the last pool_ranks ranks of every stream) are not bound to a
  // workgroup: a few workgroups at the end of the grid draw them from counters, one queue per XCD (heaviest first),
  // for as long as there are any, so that an XCD that reaches its last workgroups earlier takes more of them.
  int pool_ranks;    // 0: every workgroup has its fixed query group
  int32_t* ticket;   // one counter per XCD, kTicketStride entries apart, zero at launch
  float scale;   // softmax scale
  // few query tiles over many key rows: n_split workgroups share the tile list of one (kv stream, head group,
  // query group) and leave partial results, which prefill_split_merge_kernel combines
  int n_split;      // 1: no split
  float* part_acc;  // [workgroup, split, wavefront, 32 rows, D]
  float* part_ml;   // [workgroup, split, wavefront, 32 rows, 2] running maximum (base-2 exponent) and row sum
  // packed tiles of chunks shorter than a granule: rows more than t_long tokens behind a query group come from the
  // lists of long-lived rows (long_rows_kernel), gathered row by row; NULL = every row is walked granule by granule
  const int32_t* long_rows;    // [streams, 2, long_cap]: list A (rows every later query sees), list B (rows with a last query)
  const int32_t* long_lim;     // [streams, 2, long_cap]
  const int32_t* long_before;  // [streams, 2, n_gran + 1] entries of A / of B before every granule
  const int32_t* long_alive;   // [streams, n_rtile] first entry of B that a query of the 64-token region tile may see
  int long_cap, n_gran, n_rtile, t_long;
};

// workgroup index -> (kv stream, head group, rank of the query group; heavy query groups come first)
__device__ __forceinline__ void map_workgroup(const PrefillArgs& a, int bid, int& ks, int& hg, int& rank) {
  if (a.xcd_mode) {
    int x = bid & 7;
    int j = bid >> 3;
    int n_x = (a.B * a.Hkv / 8) * a.n_hg;
    int sl = j % n_x;
    rank = j / n_x;
    ks = x + 8 * (sl / a.n_hg);
    hg = sl % a.n_hg;
  } else {
    int ns = a.B * a.Hkv * a.n_hg;
    int sidx = bid % ns;
    rank = bid / ns;
    ks = sidx / a.n_hg;
    hg = sidx % a.n_hg;
  }
}

// ---------------------------------------------------------------------------------------------------
// fp32 / generic kernel: 64 lanes = 64 query rows, key sub-tiles of 32 rows staged in LDS as fp32.
// ---------------------------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float load_as_f32(const T* p);
template <>
__device__ __forceinline__ float load_as_f32<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float load_as_f32<uint16_t>(const uint16_t* p) { return bf16_bits_to_f32(*p); }

template <typename T>
__device__ __forceinline__ void store_from_f32(T* p, float x);
template <>
__device__ __forceinline__ void store_from_f32<float>(float* p, float x) { *p = x; }
template <>
__device__ __forceinline__ void store_from_f32<uint16_t>(uint16_t* p, float x) { *p = f32_to_bf16_bits(x); }

template <typename T, int D>
__global__ __launch_bounds__(64) void prefill_simple_kernel(PrefillArgs a) {
  constexpr int SUB = D > 128 ? 16 : 32;  // (the staged K and V rows stay within the static LDS limit)
  __shared__ float Ks[SUB][D];
  __shared__ float Vs[SUB][D];
  __shared__ float Ss[SUB][kWave];
  __shared__ int limk[SUB];

  const int lane = threadIdx.x;
  const int qt = a.qt_last - (int)blockIdx.x;  // heavy query tiles first
  const int bh = blockIdx.y;
  const int b = bh / a.Hq, hq = bh % a.Hq, hkv = hq / a.n_rep;
  const int stream = b * a.Hkv + hkv;
  const int32_t* lim = a.tok_lim + (int64_t)stream * a.N;
  const T* qp = static_cast<const T*>(a.q) + b * a.qs_b + hq * a.qs_h;
  const T* kp = static_cast<const T*>(a.k) + b * a.ks_b + hkv * a.ks_h;
  const T* vp = static_cast<const T*>(a.v) + b * a.vs_b + hkv * a.vs_h;
  T* op = static_cast<T*>(a.o) + b * a.os_b + hq * a.os_h;

  const int m = qt * kTile + lane;  // region token of this lane
  const bool row_ok = m >= a.r_begin && m < a.r_end;
  const int r0 = max(qt * kTile, a.r_begin);

  float qv[D], acc[D];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    qv[d] = row_ok ? load_as_f32<T>(qp + (int64_t)(m - a.r_begin) * a.qs_l + d) : 0.f;
    acc[d] = 0.f;
  }
  float m_run = -INFINITY, l_run = 0.f;

  const int last_key = a.base + min(qt * kTile + kTile - 1, a.r_end - 1);
  for (int k0 = 0; k0 <= last_key; k0 += SUB) {
    // does any row of this sub-tile reach the first query of the tile?
    int key = k0 + lane;
    bool reach = lane < SUB && key < a.N && lim[key] >= r0;
    if (__ballot(reach) == 0) continue;
    __syncthreads();  // previous sub-tile fully consumed
    for (int idx = lane; idx < SUB * D; idx += kWave) {
      int r = idx / D, d = idx % D;
      int n = k0 + r;
      bool ok = n < a.N;
      Ks[r][d] = ok ? load_as_f32<T>(kp + (int64_t)n * a.ks_l + d) : 0.f;
      Vs[r][d] = ok ? load_as_f32<T>(vp + (int64_t)n * a.vs_l + d) : 0.f;
    }
    if (lane < SUB) limk[lane] = key < a.N ? lim[key] : -1;
    __syncthreads();

    float tmax = -INFINITY;
    for (int j = 0; j < SUB; ++j) {
      float dot = 0.f;
#pragma unroll
      for (int d = 0; d < D; ++d) dot = fmaf(qv[d], Ks[j][d], dot);
      int n = k0 + j;
      bool vis = row_ok && n - a.base <= m && m <= limk[j];
      float s = vis ? dot * a.scale : -INFINITY;
      Ss[j][lane] = s;
      tmax = fmaxf(tmax, s);
    }
    float m_new = fmaxf(m_run, tmax);
    if (m_new != -INFINITY) {
      float alpha = expf(m_run - m_new);
      l_run *= alpha;
#pragma unroll
      for (int d = 0; d < D; ++d) acc[d] *= alpha;
      for (int j = 0; j < SUB; ++j) {
        float p = expf(Ss[j][lane] - m_new);
        l_run += p;
#pragma unroll
        for (int d = 0; d < D; ++d) acc[d] = fmaf(p, Vs[j][d], acc[d]);
      }
      m_run = m_new;
    }
  }
  if (row_ok) {
    float inv = 1.f / l_run;
#pragma unroll
    for (int d = 0; d < D; ++d) store_from_f32<T>(op + (int64_t)(m - a.r_begin) * a.os_l + d, acc[d] * inv);
  }
}

// ---------------------------------------------------------------------------------------------------
// bf16 MFMA kernel.
//
// Workgroup = 8 wavefronts = (hpw q heads of one kv head) x (qpw query tiles of 64 rows) x (2 halves of 32
// rows); every wavefront owns 32 query rows of one q head and all wavefronts share each 64-key K / V tile
// through LDS.  With 256 registers per lane two wavefronts share a SIMD, so that the vector ALU work of
// one (exponentials) runs under the matrix instructions of the other.
//
// K / V tiles travel global -> LDS without passing through registers (global_load_lds, 16 bytes per lane),
// double buffered, row major with 256-byte rows whose 16-byte chunks are XOR-swizzled (the lane supplies
// the global address, so the permutation costs nothing) to keep the operand reads free of bank conflicts.
//
// Scores are computed transposed, S^T = K Q^T (A operand = K rows from LDS, B operand = Q from registers),
// so a lane holds 16 keys of ONE query per accumulator and the softmax row reductions stay inside the
// lane (one cross-lane exchange with lane ^ 32).  The exponentials leave the accumulators already in the
// B-operand layout of O^T = V^T P^T; its A operand V^T comes from the row-major V tile through
// ds_read_b64_tr_b16, which hands every lane 4 consecutive keys of one head dimension.
//
// The running maximum is only raised when a row maximum exceeds it by more than kRescaleSlack (base-2
// exponent); until then probabilities may exceed 1 (at most 2^kRescaleSlack), which fp32 sums and bf16
// operands hold without loss, and O is not touched.
// ---------------------------------------------------------------------------------------------------
constexpr float kRescaleSlack = 8.0f;
constexpr int kPrefillWaves = 8;
constexpr int kMaxSplit = 32;  // workgroups that may share one tile list
constexpr int kMaxDevices = 64;

// both halves of the wavefront get max / sum over lane and lane ^ 32 (one cross-half swap, no LDS round trip)
__device__ __forceinline__ float half_swap_max(float v) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum(float v) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
constexpr int kWin = 1024;  // key tiles whose visit list is built at once

template <int D>
struct PrefillSmem {
  uint16_t k[4][kTile * D];  // tile j of the visit list in k[j & 3]
  uint16_t v[4][kTile * D];
  int limk[8][kTile];        // row limits of tile j in limk[j & 7]
  int posk[8][kTile];        // packed tiles: region token of every key row (a row is visible up to limk and from posk on);
                             // tiles gathered from the long-lived rows: the cache row of every key row
  int4 vlist[kWin];  // visited key tiles of the current window: {tile, max limit, min limit, -}
                     // packed tiles: the four 16-row granules of the tile ({id | mask flag, id, id, id}, -1 = none)
  int vcount;
  int ticket;  // drawn pool item of this workgroup (-1: none left) and the queue it came from
  int queue;
};
constexpr int kGranPerTile = kTile / kGranule;
constexpr int kPackedMaskFlag = 1 << 30;  // on the first granule id of a packed tile: some score of the tile is masked
constexpr int kFarTileFlag = 1 << 29;     // ... the entry is a tile of long-lived rows: 64 list entries from the second field on

// kUniform: the wavefronts are the q heads of ONE query tile (GQA groups of 4 and more), so every tile of
// the visit list is visited by every wavefront and the tile loop has no per-wavefront branches.
// kPacked (kMode 1 and 2, with kUniform, for chunks shorter than a tile): a tile is assembled from four 16-row granules taken
// from anywhere in the key rows.  Granules no query of the workgroup sees are left out, granules every query of
// the workgroup sees without a mask are packed among themselves and the rest (diagonal, partly visible, the remainder of the
// first kind, padding) into tiles that go through the element mask.  The softmax does not care about the order
// of the keys, so nothing else changes; without it a tile with one visible 16- or 32-row chunk costs a whole tile.
// (kMode: 0 whole tiles, 1 packed tiles, 2 packed tiles with the rows far behind a query gathered from the lists of
// long-lived rows)
template <int D, bool kUniform, int kMode>
__device__ __forceinline__ void prefill_mfma_item(const PrefillArgs& a, unsigned char* smem_raw, int bid, int split, int ks,
                                                  int hg, int rank) {
  constexpr bool kPacked = kMode != 0;
  constexpr bool kFar = kMode == 2;
  static_assert(!kPacked || kUniform, "packed tiles are walked by every wavefront of the workgroup");
  constexpr int OCT = D / 8;                          // 16-byte chunks per row
  constexpr int N_INST = kTile * OCT / kWave;         // 1 KiB global->LDS transfers per tile
  constexpr int DMA_PER_WAVE = (N_INST + kPrefillWaves - 1) / kPrefillWaves;  // ... per wavefront and tensor (with rows
                                                      // of 64 bytes a tile is four transfers: wavefronts 0-3 issue one each)
  constexpr int DSTEPS = D / 16;
  constexpr int DT = D / 32;
  constexpr int kHalf = kTile / 2;
  static_assert(DMA_PER_WAVE >= 1 && N_INST % DMA_PER_WAVE == 0, "tile rows are split over the wavefronts in 1 KiB transfers");
  // first tile row of this wavefront's transfers -> its granule of a packed tile
  constexpr int kRowsPerInst = kWave / OCT;

  PrefillSmem<D>& sm = *reinterpret_cast<PrefillSmem<D>*>(smem_raw);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform, and the compiler may know it
  const int sub = wave & 3;    // which (head, query tile) of the workgroup; wavefronts sub and sub + 4 share a SIMD
  const int half = wave >> 2;  // which 32 rows of the query tile
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int hl = lane >> 5;

  const int qg = a.n_qg - 1 - rank;  // heavy query groups first
  const int b = ks / a.Hkv, hkv = ks % a.Hkv;
  const int hq = hkv * a.n_rep + hg * a.hpw + (sub % a.hpw);
  const int qt_lo = a.qt_first + qg * a.qpw;
  const int qt_hi = min(qt_lo + a.qpw - 1, a.qt_last);
  const int my_qt = qt_lo + sub / a.hpw;
  const bool wave_live = my_qt <= qt_hi;
  const int q0 = my_qt * kTile + half * kHalf;  // region token of this wavefront's first row

  const int2* tl = a.tile_lim + (int64_t)ks * a.Tk;
  const int32_t* lim = a.tok_lim + (int64_t)ks * a.N;
  const uint16_t* kp = static_cast<const uint16_t*>(a.k) + b * a.ks_b + hkv * a.ks_h;
  const uint16_t* vp = static_cast<const uint16_t*>(a.v) + b * a.vs_b + hkv * a.vs_h;

  // first / last query token of the group, of this wavefront's query tile and of its 32 rows, and the last
  // key tile the group / the query tile may see
  const int r0_group = max(qt_lo * kTile, a.r_begin);
  const int rlast_group = min(qt_hi * kTile + kTile - 1, a.r_end - 1);
  const int tile_r0 = max(my_qt * kTile, a.r_begin);
  const int tile_rlast = min(my_qt * kTile + kTile - 1, a.r_end - 1);
  const int my_r0 = max(q0, a.r_begin);
  const int my_rlast = min(q0 + kHalf - 1, a.r_end - 1);
  const int kt_end_group = (a.base + rlast_group) / kTile;
  const int my_kt_end = (a.base + tile_rlast) / kTile;

  // Rows more than t_long tokens behind the group's first query: only the stream's long-lived rows can be visible
  // there (long_rows_kernel).  Below near_row0, the row from which the group walks granule by granule, lie the first
  // n_far_a entries of list A and the first b_hi of list B, of which those before b_lo are seen by nobody here.
  const bool far_mode = kFar;
  int near_row0 = 0, n_far_a = 0, b_lo = 0, b_hi = 0;
  const int32_t* lrows = nullptr;
  const int32_t* llim = nullptr;
  if (far_mode) {
    near_row0 = max(0, a.base + r0_group - a.t_long) & ~(kGranule - 1);
    const int32_t* bef = a.long_before + (int64_t)ks * 2 * (a.n_gran + 1) + near_row0 / kGranule;
    n_far_a = __builtin_amdgcn_readfirstlane(bef[0]);
    b_hi = __builtin_amdgcn_readfirstlane(bef[a.n_gran + 1]);
    b_lo = __builtin_amdgcn_readfirstlane(a.long_alive[(int64_t)ks * a.n_rtile + r0_group / kTile]);
    b_lo = min(b_lo, b_hi);
    lrows = a.long_rows + (int64_t)ks * 2 * a.long_cap;
    llim = a.long_lim + (int64_t)ks * 2 * a.long_cap;
  }
  const int n_far_ta = (n_far_a + kTile - 1) / kTile;  // gathered tiles of list A, then of list B
  const int n_far_tiles = n_far_ta + (b_hi - b_lo + kTile - 1) / kTile;

  // ---- wavefront 0 asks for the tile summaries of the first kEarly * 64 key tiles before anything else is requested:
  // memory operations complete in the order of their issue, so the wait for these (a trip to L2) does not include
  // the Q rows (a trip to HBM), which stay in flight while the visit list is built and the first tiles are requested.
  constexpr int kEarly = 8;
  int2 tl_early[kEarly];
  if (!kPacked && wave == 0) {
#pragma unroll
    for (int j = 0; j < kEarly; ++j) tl_early[j] = tl[min(j * kWave + lane, kt_end_group)];
  }

  // ---- Q fragments: B operand, lane (query l32, k-group hl) --------------------------------------
  bf16x8 qreg[DSTEPS];
  {
    const uint16_t* qp = static_cast<const uint16_t*>(a.q) + b * a.qs_b + hq * a.qs_h;
    int row = min(max(q0 + l32, a.r_begin), a.r_end - 1) - a.r_begin;
    if (!wave_live) row = 0;
    const uint4* rp = reinterpret_cast<const uint4*>(qp + (int64_t)row * a.qs_l + hl * 8);
#pragma unroll
    for (int s = 0; s < DSTEPS; ++s) qreg[s] = __builtin_bit_cast(bf16x8, rp[s * 2]);
  }

  f32x16 oacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.f;
  float m_run = -INFINITY;
  float l_run = 0.f;
  const float c = a.scale * 1.4426950408889634f;

  // V rows in LDS: the transposing read of a half wavefront covers 4 consecutive keys x 32 head dimensions (64 bytes
  // of each row).  The 16-byte chunks of a row are permuted so that these four pieces fall into the four quarters of
  // the 64 LDS banks: rows of 256 bytes (one row = all banks) move by a quarter per row, rows of 128 bytes (two rows
  // = all banks) by a quarter per pair of rows.
  // (rows of 64 bytes: four rows = all banks and the four pieces of a read are one contiguous 256 bytes)
  auto v_swizzle = [](int row) { return OCT >= 16 ? (row & 3) << 2 : OCT >= 8 ? ((row >> 1) & 1) << 2 : 0; };
  // global -> LDS, one 64-key tile of K or of V; rows beyond N repeat row N-1 (their scores are masked,
  // so their probabilities are exactly 0 and a finite V row contributes nothing).  The lane's share of a
  // tile sits at fixed offsets from the tile's first row, computed once.
  int koff[DMA_PER_WAVE], voff[DMA_PER_WAVE];
#pragma unroll
  for (int j = 0; j < DMA_PER_WAVE; ++j) {
    const int q = (wave * DMA_PER_WAVE + j) * kWave + lane;  // chunk slot in the LDS tile
    const int row = q / OCT, pos = q % OCT;
    // (packed tiles: this wavefront's 8 rows of a tile lie in one granule; the offset counts from its first row)
    const int srow = kPacked ? row % kGranule : row;
    koff[j] = int(srow * a.ks_l + (pos ^ (row % OCT)) * 8);
    voff[j] = int(srow * a.vs_l + (pos ^ v_swizzle(row)) * 8);
  }
  auto issue_rows = [&](const uint16_t* base, int64_t stride, const int (&off)[DMA_PER_WAVE], uint16_t* dst, int kt,
                        bool is_v) {
    if (kt * kTile + kTile <= a.N) {
      const uint16_t* tb = base + (int64_t)kt * kTile * stride;  // uniform
#pragma unroll
      for (int j = 0; j < DMA_PER_WAVE; ++j) {
        const int inst = wave * DMA_PER_WAVE + j;
        if (inst < N_INST)
          __builtin_amdgcn_global_load_lds(tb + (int)off[j], (uint32_t __attribute__((address_space(3)))*)(dst + inst * kWave * 8), 16, 0, 0);
      }
    } else {
#pragma unroll
      for (int j = 0; j < DMA_PER_WAVE; ++j) {
        const int inst = wave * DMA_PER_WAVE + j;  // uniform
        const int q = inst * kWave + lane;
        const int row = q / OCT, pos = q % OCT;
        const int n = min(kt * kTile + row, a.N - 1);
        const int chunk = is_v ? pos ^ v_swizzle(row) : pos ^ (row % OCT);
        if (inst < N_INST)
          __builtin_amdgcn_global_load_lds(base + (int64_t)n * stride + chunk * 8,
                                           (uint32_t __attribute__((address_space(3)))*)(dst + inst * kWave * 8), 16, 0, 0);
      }
    }
  };
  // K tile and the visibility limits of its rows; the limits go to slot (list index & 7)
  auto issue_k = [&](int kt, int buf, int slot, bool need_lim) {
    issue_rows(kp, a.ks_l, koff, sm.k[buf], kt, false);
    // (asynchronous like the tile itself; rows beyond N are later than every query, which masks them whatever
    // limit they get, so their address is clamped)
    if (need_lim && wave == 0)
      __builtin_amdgcn_global_load_lds(lim + min(kt * kTile + lane, a.N - 1),
                                       (uint32_t __attribute__((address_space(3)))*)(&sm.limk[slot][0]), 4, 0, 0);
  };
  auto issue_v = [&](int kt, int buf) { issue_rows(vp, a.vs_l, voff, sm.v[buf], kt, true); };
  // packed tiles: the wavefront's 8 rows of the tile come from granule (wave / 2) of the list entry; a missing
  // granule (padding) repeats granule 0, whose rows the limit -1 masks
  auto issue_rows_p = [&](const uint16_t* base, int64_t stride, const int (&off)[DMA_PER_WAVE], uint16_t* dst, int gid,
                          bool is_v) {
    if (gid < 0) gid = 0;
    if ((gid + 1) * kGranule <= a.N) {
      const uint16_t* tb = base + (int64_t)gid * kGranule * stride;  // uniform
#pragma unroll
      for (int j = 0; j < DMA_PER_WAVE; ++j) {
        const int inst = wave * DMA_PER_WAVE + j;
        if (inst < N_INST)
          __builtin_amdgcn_global_load_lds(tb + (int)off[j], (uint32_t __attribute__((address_space(3)))*)(dst + inst * kWave * 8), 16, 0, 0);
      }
    } else {
#pragma unroll
      for (int j = 0; j < DMA_PER_WAVE; ++j) {
        const int inst = wave * DMA_PER_WAVE + j;  // uniform
        const int q = inst * kWave + lane;
        const int row = q / OCT, pos = q % OCT;
        const int n = min(gid * kGranule + row % kGranule, a.N - 1);
        const int chunk = is_v ? pos ^ v_swizzle(row) : pos ^ (row % OCT);
        if (inst < N_INST)
          __builtin_amdgcn_global_load_lds(base + (int64_t)n * stride + chunk * 8,
                                           (uint32_t __attribute__((address_space(3)))*)(dst + inst * kWave * 8), 16, 0, 0);
      }
    }
  };
  // a tile of the list of long-lived rows: the cache row of every tile row is in posk[slot] (requested a step ahead)
  auto issue_rows_far = [&](const uint16_t* base, int64_t stride, uint16_t* dst, int slot, bool is_v) {
#pragma unroll
    for (int j = 0; j < DMA_PER_WAVE; ++j) {
      const int inst = wave * DMA_PER_WAVE + j;  // uniform
      const int q = inst * kWave + lane;
      const int row = q / OCT, pos = q % OCT;
      const int n = max(0, min(sm.posk[slot][row & (kTile - 1)], a.N - 1));  // (padding entries hold INT_MAX and the limit -1)
      const int chunk = is_v ? pos ^ v_swizzle(row) : pos ^ (row % OCT);
      if (inst < N_INST)
        __builtin_amdgcn_global_load_lds(base + (int64_t)n * stride + chunk * 8,
                                         (uint32_t __attribute__((address_space(3)))*)(dst + inst * kWave * 8), 16, 0, 0);
    }
  };
  // (id0: the first field of the list entry, with its flags; mine: this wavefront's granule of the tile, or the first
  // list entry of a gathered tile; idx: the entry's place in the list)
  auto issue_k_p = [&](int id0, int mine, int idx, int buf, int slot) {
    if (kFar && (id0 & kFarTileFlag)) {
      issue_rows_far(kp, a.ks_l, sm.k[buf], slot, false);
      if ((id0 & kPackedMaskFlag) && wave == 0) {
        int ln = lane;
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("" : "+v"(ln));
#endif
        __builtin_amdgcn_global_load_lds(llim + mine + ln,
                                         (uint32_t __attribute__((address_space(3)))*)(&sm.limk[slot][0]), 4, 0, 0);
      }
      return;
    }
    issue_rows_p(kp, a.ks_l, koff, sm.k[buf], mine, false);
    if ((id0 & kPackedMaskFlag) && wave == 0) {
      // limits and region tokens of the 64 rows, for the element mask (asynchronous like the tile itself).
      // (The lane id is taken afresh so that nothing derived from it has to live across the tile loop.)
      int ln = lane;
#if defined(__HIP_DEVICE_COMPILE__)
      asm volatile("" : "+v"(ln));
#endif
      int gid = reinterpret_cast<const int*>(&sm.vlist[idx])[ln >> 4];
      if ((ln >> 4) == 0) gid &= ~kPackedMaskFlag;
      const int row = gid * kGranule + (ln & (kGranule - 1));
      const bool real = gid >= 0 && row < a.N;
      const int32_t* src = real ? lim + row : a.tok_lim + (int64_t)a.B * a.Hkv * a.N;  // (the entry that holds -1)
      __builtin_amdgcn_global_load_lds(src, (uint32_t __attribute__((address_space(3)))*)(&sm.limk[slot][0]), 4, 0, 0);
      sm.posk[slot][ln] = real ? row - a.base : 0x7fffffff;
    }
  };
  auto issue_v_p = [&](int id0, int mine, int buf, int slot) {
    if (kFar && (id0 & kFarTileFlag)) {
      issue_rows_far(vp, a.vs_l, sm.v[buf], slot, true);
      return;
    }
    issue_rows_p(vp, a.vs_l, voff, sm.v[buf], mine, true);
  };

  auto k_frag = [&](const uint16_t* Kt, int kb, int s) {
    const int row = kb * 32 + l32;
    const int chunk = (s * 2 + hl) ^ (row % OCT);
    return *reinterpret_cast<const bf16x8*>(Kt + row * D + chunk * 8);
  };
  // ds_read_b64_tr_b16: within 16 lanes, lane r reads 4 dims of key (K0 + r / 4) starting at dim
  // D0 + 4 * (r % 4) and receives keys K0 .. K0 + 3 of dim D0 + r.
  const int r16 = lane & 15;
  const int dsel = (lane >> 4) & 1;
  auto v_frag = [&](const uint16_t* Vt, int t, int dt) {
    const int chunk0 = dt * 4 + dsel * 2 + ((r16 & 3) >> 1);
    const int half4 = (r16 & 1) * 4;
    const int row_lo = t * 16 + hl * 4 + (r16 >> 2);
    const int row_hi = row_lo + 8;
    const uint16_t* pl = Vt + row_lo * D + ((chunk0 ^ v_swizzle(row_lo)) * 8) + half4;
    const uint16_t* ph = Vt + row_hi * D + ((chunk0 ^ v_swizzle(row_hi)) * 8) + half4;
    bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4 __attribute__((address_space(3)))*)pl);
    bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4 __attribute__((address_space(3)))*)ph);
    bf16x8 va = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return va;
  };

  // ---- S^T = K Q^T -----------------------------------------------------------------------------------
  auto qk_tile = [&](int buf, f32x16 (&sacc)[2]) {
    const uint16_t* Kt = sm.k[buf];
#pragma unroll
    for (int s = 0; s < DSTEPS; ++s) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        bf16x8 ka = k_frag(Kt, kb, s);
        if (s == 0) {
          const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qreg[s], z, 0, 0, 0);
        } else {
          sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qreg[s], sacc[kb], 0, 0, 0);
        }
      }
    }
  };
  // The scores of the first tile of a list have nothing to run under: every K fragment is requested before the first
  // matrix instruction, so that the LDS latency is paid once and not once per pair of instructions.
  auto qk_tile_first = [&](int buf, f32x16 (&sacc)[2]) {
    const uint16_t* Kt = sm.k[buf];
    constexpr int N_QK = 2 * DSTEPS;
    constexpr int AHEAD = N_QK < 8 ? N_QK : 8;  // fragments in flight
    bf16x8 kf[AHEAD];
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) kf[i] = k_frag(Kt, i & 1, i >> 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < N_QK; ++i) {
      const int s = i >> 1, kb = i & 1;
      if (s == 0) {
        const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i % AHEAD], qreg[s], z, 0, 0, 0);
      } else {
        sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i % AHEAD], qreg[s], sacc[kb], 0, 0, 0);
      }
      if (i + AHEAD < N_QK) kf[i % AHEAD] = k_frag(Kt, (i + AHEAD) & 1, (i + AHEAD) >> 1);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // ---- mask of a diagonal tile, or of a tile whose rows are not uniformly visible ---------------------
  auto mask_scores = [&](int kt, int slot, f32x16 (&sv)[2]) {
    const int qtok = q0 + l32;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        int kk = kb * 32 + g4 * 8 + hl * 4;  // key offset in tile of accumulator 4*g4
        int4 lm = *reinterpret_cast<const int4*>(&sm.limk[slot][kk]);
        const int lv[4] = {lm.x, lm.y, lm.z, lm.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          int key = kt * kTile + kk + e - a.base;  // region token of the key row (negative: older row)
          bool vis = key <= qtok && qtok <= lv[e];
          if (!vis) sv[kb][g4 * 4 + e] = -INFINITY;
        }
      }
    }
  };
  // packed tile: every key row carries its own region token
  // (a tile of long-lived rows: posk holds cache rows, and the rows from near_row0 on belong to the granule walk)
  auto mask_scores_p = [&](int slot, f32x16 (&sv)[2], bool far_tile) {
    const int qtok = q0 + l32;
    const int bound = far_tile ? near_row0 - 1 : qtok;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int kk = kb * 32 + g4 * 8 + hl * 4;
        const int4 lm = *reinterpret_cast<const int4*>(&sm.limk[slot][kk]);
        const int4 ps = *reinterpret_cast<const int4*>(&sm.posk[slot][kk]);
        const int lv[4] = {lm.x, lm.y, lm.z, lm.w};
        const int pv[4] = {ps.x, ps.y, ps.z, ps.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const bool vis = pv[e] <= bound && qtok <= lv[e];
          if (!vis) sv[kb][g4 * 4 + e] = -INFINITY;
        }
      }
    }
  };
  auto row_max = [&](const f32x16 (&sv)[2]) {
    float m = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) m = fmaxf(m, sv[kb][i]);
    return half_swap_max(m) * c;
  };
  // ---- raise the running maximum (rare): O and l shrink by 2^(old - new) ----------------------------
  auto rescale = [&](float mx) {
    float m_new = fmaxf(m_run, mx);
    float alpha = m_run == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run - m_new);
    l_run *= alpha;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[dt][i] *= alpha;
  };
  // n-th probability of the tile in the order the PV MFMAs consume them (16 keys per B operand)
  auto prob = [&](const f32x16 (&sv)[2], int n, float m_use, float& rs, bf16x8 (&pb)[4]) {
    const int t = n >> 3, i = n & 7;
    float p = __builtin_amdgcn_exp2f(fmaf(sv[t >> 1][(t & 1) * 8 + i], c, -m_use));
    rs += p;
    pb[t][i] = (__bf16)p;
  };
  // ---- plain step: probabilities, then O^T += V^T P^T ------------------------------------------------
  auto finish_tile = [&](int vbuf, const f32x16 (&sv)[2]) {
    const uint16_t* Vt = sm.v[vbuf];
    const float m_use = m_run == -INFINITY ? 0.f : m_run;
    float rs = 0.f;
    bf16x8 pb[4];
#pragma unroll
    for (int n = 0; n < 32; ++n) prob(sv, n, m_use, rs, pb);
    l_run += rs;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v_frag(Vt, t, dt), pb[t], oacc[dt], 0, 0, 0);
  };
  // ---- fused step: scores of the next tile, probabilities of this one, O += P V of this one ----------
  // A matrix instruction occupies the matrix pipe for 8 passes, during which vector ALU work can issue.  The
  // step is written as slots of one MFMA followed by a slice of the exponentials, fenced so that the compiler
  // keeps the slots in this order:
  //   phase A  score MFMAs of the next tile   + probabilities of keys  0..31 of this tile
  //   phase B  O += P V for keys 0..31        + probabilities of keys 32..63
  //   phase C  O += P V for keys 32..63
  auto fused_step = [&](int kbuf_next, int vbuf, const f32x16 (&sv)[2], f32x16 (&sacc)[2]) {
    const uint16_t* Kt = sm.k[kbuf_next];
    const uint16_t* Vt = sm.v[vbuf];
    constexpr int N_QK = 2 * DSTEPS;         // score MFMAs
    constexpr int N_PV = 4 * DT;             // PV MFMAs
    constexpr int VA = 16 / N_QK > 0 ? 16 / N_QK : 1;  // probabilities per slot in phase A
    constexpr int VB = 16 / (N_PV / 2);      // ... in phase B
    const float m_use = m_run == -INFINITY ? 0.f : m_run;
    float rs = 0.f;
    bf16x8 pb[4];
    int n = 0;
    __builtin_amdgcn_sched_barrier(0);
    // LDS operands are fetched two slots ahead of the MFMA that consumes them (rings of three fragments)
    auto k_at = [&](int i) { return k_frag(Kt, i & 1, i >> 1); };   // i-th score MFMA: (kb, s) = (i & 1, i >> 1)
    auto v_at = [&](int i) { return v_frag(Vt, i / DT, i % DT); };  // i-th PV MFMA: (t, dt) = (i / DT, i % DT)
    bf16x8 kf[3], vf[3];
    kf[0] = k_at(0);
    kf[1] = k_at(1);
#pragma unroll
    for (int i = 0; i < N_QK; ++i) {
      const int s = i >> 1, kb = i & 1;
      if (i + 2 < N_QK) {
        kf[(i + 2) % 3] = k_at(i + 2);
      } else {
        vf[(i + 2 - N_QK) % 3] = v_at(i + 2 - N_QK);
      }
      if (s == 0) {
        const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i % 3], qreg[s], z, 0, 0, 0);
      } else {
        sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i % 3], qreg[s], sacc[kb], 0, 0, 0);
      }
      if (n < 16) {
#pragma unroll
        for (int e = 0; e < VA; ++e) prob(sv, n++, m_use, rs, pb);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (; n < 16;) prob(sv, n++, m_use, rs, pb);
#pragma unroll
    for (int i = 0; i < N_PV; ++i) {
      const int t = i / DT, dt = i % DT;
      if (i + 2 < N_PV) vf[(i + 2) % 3] = v_at(i + 2);
      oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[i % 3], pb[t], oacc[dt], 0, 0, 0);
      if (t < 2) {
#pragma unroll
        for (int e = 0; e < VB; ++e) prob(sv, n++, m_use, rs, pb);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    l_run += rs;
  };

  // Scores of the tile that the next step turns into probabilities.
  f32x16 sacc[2];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int i = 0; i < 16; ++i) sacc[kb][i] = 0.f;

  // Visit list of a window of whole tiles: wavefront 0 compacts the tiles some query of the group sees.  (The first
  // window is built ahead of the window loop, from the summaries requested at the top of the kernel, so that those do
  // not stay in registers through the tile loop.)
  auto compact_round = [&](int t, int2 val, int& count) {
    const bool v = t <= kt_end_group && val.x >= r0_group;
    const uint64_t bits = __ballot(v);
    if (v) sm.vlist[count + __builtin_popcountll(bits & ((uint64_t(1) << lane) - 1))] = make_int4(t, val.x, val.y, 0);
    count += __builtin_popcountll(bits);
  };
  auto build_list = [&](int w0, bool first) {
    // (rounds beyond the last tile the group may see are skipped: the tests on j are uniform)
    int2 vals[kWin / kWave];
#pragma unroll
    for (int j = 0; j < kWin / kWave; ++j) {
      if (w0 + j * kWave <= kt_end_group) {
        if (first && j < kEarly) {
          vals[j] = tl_early[j];
        } else {
          vals[j] = tl[min(w0 + j * kWave + lane, kt_end_group)];
        }
      }
    }
    int count = 0;
#pragma unroll
    for (int j = 0; j < kWin / kWave; ++j)
      if (w0 + j * kWave <= kt_end_group) compact_round(w0 + j * kWave + lane, vals[j], count);
    if (lane == 0) sm.vcount = count;
  };
  if (!kPacked && wave == 0) {
    if (kt_end_group < kEarly * kWave) {
      // every tile summary the list needs was requested at the top: nothing else is loaded here, and the wait for
      // the summaries leaves the Q rows in flight
      int count = 0;
#pragma unroll
      for (int j = 0; j < kEarly; ++j)
        if (j * kWave <= kt_end_group) compact_round(j * kWave + lane, tl_early[j], count);
      if (lane == 0) sm.vcount = count;
    } else {
      build_list(0, true);
    }
  }

  // (packed tiles: the window counts granules, and leaves room for the one tile the packing can add)
  const int g_end_group = (a.base + rlast_group) / kGranule;
  const int win_last = kPacked ? g_end_group : kt_end_group;
  constexpr int kWinStep = kPacked ? (kWin - 1) * kGranPerTile : kWin;
  int f0 = 0;                                // first tile of the long-lived rows in this window
  bool far_win = far_mode && n_far_tiles > 0;  // windows of gathered tiles come first, then the granule walk
  for (int w0 = far_mode ? near_row0 / kGranule : 0; w0 <= win_last;) {
    // ---- visit list of this window: wavefront 0 compacts the tiles some query tile of the group sees ----
    // far_cnt gathered tiles at the head of the list; the granule walk joins the window that holds the last of them
    // when its tiles fit behind (the usual case: one pass of the tile pipeline per workgroup)
    int far_cnt = 0;
    bool with_near = !far_win;
    if (kFar && far_win) {
      far_cnt = min(kWin - 1, n_far_tiles - f0);
      const int n_near = g_end_group - w0 + 1;  // granules of the walk
      with_near = f0 + far_cnt == n_far_tiles && n_near <= kWinStep &&
                  far_cnt + (n_near + kGranPerTile - 1) / kGranPerTile + 1 <= kWin - 1;
    }
    if (kFar && far_win && wave == 0) {
      // gathered tiles [f0, f0 + count): whole tiles of list A need no mask (every query sees their rows, and they
      // lie below near_row0); the last one of A and the tiles of B go through it
      const int cnt = far_cnt;
      for (int i = lane; i < cnt; i += kWave) {
        const int t = f0 + i;
        int4 d;
        if (t < n_far_ta) {
          d = make_int4(kFarTileFlag | ((t + 1) * kTile <= n_far_a ? 0 : kPackedMaskFlag), t * kTile, 0, 0);
        } else {
          d = make_int4(kFarTileFlag | kPackedMaskFlag, a.long_cap + b_lo + (t - n_far_ta) * kTile, 0, 0);
        }
        sm.vlist[i] = d;
      }
      if (lane == 0 && !with_near) sm.vcount = cnt;
    }
    if (kPacked && with_near && wave == 0) {
      // granules seen without a mask and granules that need one, each kind in its own list (staged in the tile
      // buffers, which are idle here), then four ids per tile
      int* plain_ids = reinterpret_cast<int*>(&sm.k[0][0]);
      int* mask_ids = reinterpret_cast<int*>(&sm.v[0][0]);
      const int2* gl = a.gran_lim + (int64_t)ks * a.Tk * kGranPerTile;
      const int g_hi = min(w0 + kWinStep - 1, g_end_group);
      int n_plain = 0, n_mask = 0;
      // first the 64-row tiles that somebody in the group sees (one summary per tile), then only their granules
      int* cand = reinterpret_cast<int*>(&sm.k[1][0]);
      const int t_lo = w0 / kGranPerTile, t_hi = g_hi / kGranPerTile;
      int n_c = 0;
      for (int tb = t_lo; tb <= t_hi; tb += 8 * kWave) {
        int mx[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int t = tb + u * kWave + lane;
          mx[u] = t <= t_hi ? tl[t].x : -1;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const bool vis = mx[u] >= r0_group && tb + u * kWave + lane <= t_hi;
          const uint64_t bv = __ballot(vis);
          if (vis) cand[n_c + __builtin_popcountll(bv & ((uint64_t(1) << lane) - 1))] = tb + u * kWave + lane;
          n_c += __builtin_popcountll(bv);
        }
      }
      wave_lds_sync();
      for (int cb = 0; cb < n_c; cb += kWave) {
        const int t = cb + lane < n_c ? cand[cb + lane] : -1;
        int2 vals[kGranPerTile];
#pragma unroll
        for (int u = 0; u < kGranPerTile; ++u) vals[u] = t >= 0 ? gl[t * kGranPerTile + u] : make_int2(-1, -1);
#pragma unroll
        for (int u = 0; u < kGranPerTile; ++u) {
          const int g = t * kGranPerTile + u;
          const bool vis = t >= 0 && g >= w0 && g <= g_hi && vals[u].x >= r0_group;
          const int last_pos = g * kGranule + kGranule - 1 - a.base;
          const bool plain = vis && vals[u].y >= rlast_group && last_pos <= r0_group && (g + 1) * kGranule <= a.N;
          const bool masked = vis && !plain;
          const uint64_t bp = __ballot(plain), bm = __ballot(masked);
          const uint64_t below = (uint64_t(1) << lane) - 1;
          if (plain) plain_ids[n_plain + __builtin_popcountll(bp & below)] = g;
          if (masked) mask_ids[n_mask + __builtin_popcountll(bm & below)] = g;
          n_plain += __builtin_popcountll(bp);
          n_mask += __builtin_popcountll(bm);
        }
      }
      wave_lds_sync();
      const int n_pt = n_plain / kGranPerTile;
      const int left = n_plain - n_pt * kGranPerTile;  // these join the masked kind
      if (lane < left) mask_ids[n_mask + lane] = plain_ids[n_pt * kGranPerTile + lane];
      n_mask += left;
      wave_lds_sync();
      const int n_mt = (n_mask + kGranPerTile - 1) / kGranPerTile;
      for (int i = lane; i < n_pt + n_mt; i += kWave) {
        int4 d;
        if (i < n_pt) {
          const int* p = plain_ids + i * kGranPerTile;
          d = make_int4(p[0], p[1], p[2], p[3]);
        } else {
          const int o = (i - n_pt) * kGranPerTile;
          d.x = mask_ids[o] | kPackedMaskFlag;
          d.y = o + 1 < n_mask ? mask_ids[o + 1] : -1;
          d.z = o + 2 < n_mask ? mask_ids[o + 2] : -1;
          d.w = o + 3 < n_mask ? mask_ids[o + 3] : -1;
        }
        sm.vlist[far_cnt + i] = d;
      }
      if (lane == 0) sm.vcount = far_cnt + n_pt + n_mt;
    }
    if (!kPacked && wave == 0 && w0 > 0) build_list(w0, false);
    __syncthreads();
    int n_vis = __builtin_amdgcn_readfirstlane(sm.vcount);
    int j0 = 0;  // first list entry of this workgroup's share
    if (a.n_split > 1) {
      const int per = (n_vis + a.n_split - 1) / a.n_split;
      j0 = split * per;
      n_vis = max(0, min(per, n_vis - j0));
    }
    if (n_vis > 0) {
      // The list entries are the same for every lane: they are kept in scalar registers.
      // Tile j of the list: the matrix pipe computes the scores of tile j+1 while the vector ALU turns those of
      // tile j into probabilities; then O += P V for tile j.  Buffers: K tile j in k[j & 3], V tile j in
      // v[j & 3], row limits of tile j in limk[j & 7].
      auto entry = [&](int j, int& kt, int& emax, int& emin) {
        const int4 e = sm.vlist[j0 + j];
        kt = __builtin_amdgcn_readfirstlane(e.x);
        emax = __builtin_amdgcn_readfirstlane(e.y);
        emin = __builtin_amdgcn_readfirstlane(e.z);
      };
      // the element mask is only evaluated on diagonal tiles and on tiles with mixed visibility
      auto group_needs_lim = [&](int kt, int emin) { return kt * kTile + kTile - 1 - a.base > r0_group || emin < rlast_group; };
      auto visits = [&](int kt, int emax) { return kUniform || (wave_live && kt <= my_kt_end && emax >= tile_r0); };

      // One step handles two tiles of the list (2s, 2s + 1) between two workgroup barriers.  At its start the
      // K tiles 2s + 1, 2s + 2 and the V tiles 2s, 2s + 1 are in LDS and the scores of tile 2s in registers; the
      // step puts K tiles 2s + 3, 2s + 4 and V tiles 2s + 2, 2s + 3 in flight.
      // (packed tiles: kt is the entry's first field with its flags, emax this wavefront's granule of the tile -- or
      // the first list entry of a gathered tile -- and emin the entry's place in the list)
      struct Entry {
        int kt, emax, emin;
      };
      auto read_entry = [&](int j) {
        Entry r = {0, 0, 0};
        if (j < n_vis) {
          if (kPacked) {
            const int* ep = reinterpret_cast<const int*>(&sm.vlist[j0 + j]);
            r.kt = __builtin_amdgcn_readfirstlane(ep[0]);
            // (this wavefront's granule: the one its first transferred row lies in; a wavefront without transfers
            // reads the last one and does not use it)
            const int my_gran = min(wave * DMA_PER_WAVE * kRowsPerInst / kGranule, kGranPerTile - 1);
            const int sel = (kFar && (r.kt & kFarTileFlag)) ? 1 : my_gran;
            const int mine = __builtin_amdgcn_readfirstlane(ep[sel]);
            r.emax = sel == 0 ? mine & ~kPackedMaskFlag : mine;
            r.emin = j0 + j;
          } else {
            int kt, emax, emin;
            entry(j, kt, emax, emin);
            r.kt = kt; r.emax = emax; r.emin = emin;
          }
        }
        return r;
      };
      auto load_k = [&](int j, const Entry& e) {
        if (j < n_vis) {
          if (kPacked) {
            issue_k_p(e.kt, e.emax, e.emin, j & 3, j & 7);
          } else {
            issue_k(e.kt, j & 3, j & 7, group_needs_lim(e.kt, e.emin));
          }
        }
      };
      auto load_v = [&](int j, const Entry& e) {
        if (j < n_vis) {
          if (kPacked) {
            issue_v_p(e.kt, e.emax, j & 3, j & 7);
          } else {
            issue_v(e.kt, j & 3);
          }
        }
      };
      // tile t: its scores (in sacc) become probabilities while the scores of tile t + 1 are computed, then O += P V
      auto process_tile = [&](int t, const Entry& ec, const Entry& en) {
        const bool vis_c = visits(ec.kt, ec.emax);
        // (uniform case: the last tile computes scores of a stale tile that nobody reads, which keeps the step
        // free of branches around the matrix instructions)
        const bool vis_n = kUniform || (t + 1 < n_vis && visits(en.kt, en.emax));
        if (vis_c) {
          f32x16 sv[2] = {sacc[0], sacc[1]};
          // no masked score: every key row is at or before the first query and visible to the last one
          const bool full = kPacked ? !(ec.kt & kPackedMaskFlag)
                                    : (ec.kt * kTile + kTile - 1 - a.base <= my_r0 && ec.emin >= my_rlast);
          if (!full) {
            if (kPacked) {
              mask_scores_p(t & 7, sv, kFar && (ec.kt & kFarTileFlag) != 0);
            } else {
              mask_scores(ec.kt, t & 7, sv);
            }
          }
          const float mx = row_max(sv);
          if (__ballot(mx > m_run + kRescaleSlack)) rescale(mx);
          if (kUniform) {
            fused_step((t + 1) & 3, t & 3, sv, sacc);
          } else {
            // wavefronts with different query tiles: the same pipeline, its two halves one after the other
            finish_tile(t & 3, sv);
            if (vis_n) qk_tile((t + 1) & 3, sacc);
          }
        } else if (vis_n) {
          qk_tile((t + 1) & 3, sacc);
        }
      };

      // gathered tiles: the cache rows of tile j of the window go to posk[j & 7] a step before its K rows are
      // requested (asynchronous; the step's wait and barrier make them visible to every wavefront)
      auto load_ids = [&](int j) {
        if (kFar && j < n_vis && j0 + j < far_cnt && wave == 0) {
          int ln = lane;
#if defined(__HIP_DEVICE_COMPILE__)
          asm volatile("" : "+v"(ln));
#endif
          const int start = __builtin_amdgcn_readfirstlane(sm.vlist[j0 + j].y);
          __builtin_amdgcn_global_load_lds(lrows + start + ln,
                                           (uint32_t __attribute__((address_space(3)))*)(&sm.posk[j & 7][0]), 4, 0, 0);
        }
      };
      if (kFar && j0 < far_cnt) {
#pragma unroll
        for (int j = 0; j < 5; ++j) load_ids(j);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
      }
      Entry e0 = read_entry(0), e1 = read_entry(1), e2 = read_entry(2);
      load_k(0, e0);
      load_v(0, e0);
      load_k(1, e1);
      load_v(1, e1);
      load_k(2, e2);
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
      if (visits(e0.kt, e0.emax)) qk_tile_first(0, sacc);
      __syncthreads();  // k[0] is overwritten by the first step

      for (int t = 0; t < n_vis; t += 2) {
        const Entry e3 = read_entry(t + 3), e4 = read_entry(t + 4);
        load_k(t + 3, e3);
        load_k(t + 4, e4);
        load_v(t + 2, e2);
        load_v(t + 3, e3);
        load_ids(t + 5);
        load_ids(t + 6);
        process_tile(t, e0, e1);
        if (t + 1 < n_vis) process_tile(t + 1, e1, e2);
        e0 = e2; e1 = e3; e2 = e4;
        __builtin_amdgcn_s_waitcnt(0);  // the tiles in flight have landed in LDS
        __syncthreads();                // ... for every wavefront, and the tiles of this step are no longer read
      }
    } else if (!with_near || w0 + kWinStep <= win_last) {
      __syncthreads();  // (nobody may still be reading this window's count when wavefront 0 starts the next list)
    }
    if (far_win) {
      f0 += far_cnt;
      far_win = f0 < n_far_tiles;
    }
    if (with_near) w0 += kWinStep;
  }

  // ---- a share of the tile list: the unnormalised sums, the running maximum and the row sum leave as they are ----
  if (a.n_split > 1) {
    const float l = half_swap_sum(l_run);
    const int64_t slot = ((int64_t)bid * a.n_split + split) * kPrefillWaves + wave;
    float* pa = a.part_acc + (slot * kHalf + l32) * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int d = dt * 32 + g4 * 8 + hl * 4;
        *reinterpret_cast<float4*>(pa + d) =
            make_float4(oacc[dt][g4 * 4 + 0], oacc[dt][g4 * 4 + 1], oacc[dt][g4 * 4 + 2], oacc[dt][g4 * 4 + 3]);
      }
    }
    if (hl == 0) *reinterpret_cast<float2*>(a.part_ml + (slot * kHalf + l32) * 2) = make_float2(m_run, l);
    return;
  }

  // ---- epilogue: O rows go through LDS so that every row leaves as whole 16-byte pieces ----------------
  // (all wavefronts are past the last barrier of the tile loop: the tile buffers are free)
  constexpr int kRowPitch = D * 2 + 16;  // bytes; the pad spreads the rows over the banks
  static_assert(kPrefillWaves * kHalf * kRowPitch <= sizeof(PrefillSmem<D>), "staging area fits the tile buffers");
  unsigned char* stage = smem_raw + wave * (kHalf * kRowPitch);
  {
    const float l = half_swap_sum(l_run);
    const float inv = 1.f / l;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        int d = dt * 32 + g4 * 8 + hl * 4;
        // (the hardware conversion: round to nearest even, two values per instruction)
        const bf16x4 ob = {(__bf16)(oacc[dt][g4 * 4 + 0] * inv), (__bf16)(oacc[dt][g4 * 4 + 1] * inv),
                           (__bf16)(oacc[dt][g4 * 4 + 2] * inv), (__bf16)(oacc[dt][g4 * 4 + 3] * inv)};
        const uint2 ou = __builtin_bit_cast(uint2, ob);
        const uint32_t lo = ou.x, hi = ou.y;
        *reinterpret_cast<uint2*>(stage + l32 * kRowPitch + d * 2) = make_uint2(lo, hi);
      }
    }
  }
  wave_lds_sync();
  if (wave_live) {
    uint16_t* op = static_cast<uint16_t*>(a.o) + b * a.os_b + hq * a.os_h;
    constexpr int kPieces = kHalf * OCT / kWave;  // 16-byte pieces per lane
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const int id = i * kWave + lane;
      const int row = id / OCT, piece = id % OCT;
      const int qtok = q0 + row;
      if (qtok >= a.r_begin && qtok < a.r_end) {
        // (streaming store: the output is written once and read by nobody here; it should not displace K / V tiles in L2)
        const u32x4 val = *reinterpret_cast<const u32x4*>(stage + row * kRowPitch + piece * 16);
        __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(op + (int64_t)(qtok - a.r_begin) * a.os_l + piece * 8));
      }
    }
  }
}

// One (kv stream, head group, query group) per workgroup.  The workgroups at the end of the grid (two per compute
// unit) have no query group of their own: they draw the pooled ones (the lightest of every stream) from counters for
// as long as there are any.  XCDs do not finish their fixed share at the same time (streams differ in how many keys
// their roles keep visible, and the XCDs of one device differ in speed by a few percent): those that get to the pool
// earlier take more of it.  The tile loop exists twice in the code, once for each kind of workgroup, so that the
// loop around the pooled one costs the other nothing.
template <int D, bool kUniform, int kMode = 0>
__global__ __launch_bounds__(kPrefillWaves * kWave) void prefill_mfma_kernel(PrefillArgs args) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  int bid = blockIdx.x;
  int split = 0;  // which share of the tile list (n_split > 1)
  if (args.n_split > 1) {
    split = bid % args.n_split;
    bid /= args.n_split;
  }
  if (args.pool_ranks == 0 || bid < (args.n_qg - args.pool_ranks) * args.B * args.Hkv * args.n_hg) {
    int ks, hg, rank;
    map_workgroup(args, bid, ks, hg, rank);
    prefill_mfma_item<D, kUniform, kMode>(args, smem_raw, bid, split, ks, hg, rank);
    return;
  }
  // Pooled query groups wait in one queue per XCD (that of their stream, heaviest first; every counter in a 128-byte
  // line of its own).  A workgroup empties the queue of its own XCD, whose L2 holds the stream's tiles; then it looks
  // at all counters, moves on to the fullest queue (twice at most), or ends.
  // The arguments are read afresh for every item (through a pointer the compiler cannot see through), so that none of
  // them has to stay in a register from one item to the next.
  PrefillSmem<D>& sm = *reinterpret_cast<PrefillSmem<D>*>(smem_raw);
  static_assert(sizeof(PrefillArgs) % 4 == 0, "copied in 32-bit words");
  struct ArgWords {
    uint32_t w[sizeof(PrefillArgs) / 4];
  };
  auto argp = __builtin_amdgcn_kernarg_segment_ptr();
  int q = args.xcd_mode ? (bid & 7) : 0;
  int moves = 0;  // queues of other XCDs this workgroup has moved on to (thread 0 keeps count)
  for (;;) {
    asm volatile("" : "+s"(argp));
    ArgWords aw;
#pragma unroll
    for (unsigned i = 0; i < sizeof(PrefillArgs) / 4; ++i) aw.w[i] = ((const __attribute__((opencl_constant)) uint32_t*)argp)[i];
    const PrefillArgs a = __builtin_bit_cast(PrefillArgs, aw);
    const int nq = a.xcd_mode ? 8 : 1;
    const int n_x = a.B * a.Hkv * a.n_hg / nq;  // items of one rank in one queue
    const int qlen = a.pool_ranks * n_x;
    if (threadIdx.x == 0) {
      int t = atomicAdd(a.ticket + q * kTicketStride, 1);
      if (t >= qlen && moves < 2 && nq > 1) {
        int best = -1, best_left = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int left = qlen - __hip_atomic_load(a.ticket + i * kTicketStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (left > best_left) best = i, best_left = left;
        }
        if (best >= 0) {
          q = best;
          ++moves;
          t = atomicAdd(a.ticket + q * kTicketStride, 1);
        }
      }
      sm.ticket = t < qlen ? t : -1;
      sm.queue = q;
    }
    __syncthreads();
    const int t = __builtin_amdgcn_readfirstlane(sm.ticket);
    const int q_now = __builtin_amdgcn_readfirstlane(sm.queue);
    if (t < 0) break;
    q = q_now;
    const int sl = t % n_x;
    const int ks = a.xcd_mode ? q + 8 * (sl / a.n_hg) : sl / a.n_hg;
    prefill_mfma_item<D, kUniform, kMode>(a, smem_raw, bid, split, ks, sl % a.n_hg, a.n_qg - a.pool_ranks + t / n_x);
    __syncthreads();  // the output staging of this item and the ticket are read before the next item writes LDS
  }
}

// Combines the partial results of the n_split workgroups that shared one tile list: grid = (the workgroups of the
// unsplit launch, slices of their 8 x 32 x D / 4 outputs), one thread per (wavefront, row, 4 dims).
template <int D>
__global__ __launch_bounds__(256) void prefill_split_merge_kernel(PrefillArgs a) {
  constexpr int kHalf = kTile / 2;
  constexpr int Q4 = D / 4;
  const int bid = blockIdx.x;
  int ks, hg, rank;
  map_workgroup(a, bid, ks, hg, rank);
  const int qg = a.n_qg - 1 - rank;
  const int b = ks / a.Hkv, hkv = ks % a.Hkv;
  const int qt_lo = a.qt_first + qg * a.qpw;
  const int qt_hi = min(qt_lo + a.qpw - 1, a.qt_last);
  {
    const int item = blockIdx.y * 256 + threadIdx.x;
    if (item >= kPrefillWaves * kHalf * Q4) return;
    const int wave = item / (kHalf * Q4);
    const int row = (item / Q4) % kHalf;
    const int d = (item % Q4) * 4;
    const int sub = wave & 3, half = wave >> 2;
    const int my_qt = qt_lo + sub / a.hpw;
    const int qtok = my_qt * kTile + half * kHalf + row;
    if (my_qt > qt_hi || qtok < a.r_begin || qtok >= a.r_end) return;
    const int hq = hkv * a.n_rep + hg * a.hpw + (sub % a.hpw);
    const int64_t first = ((int64_t)bid * a.n_split * kPrefillWaves + wave) * kHalf + row;  // split 0
    const int64_t step = (int64_t)kPrefillWaves * kHalf;                                       // to the next split
    // the (maximum, sum) pairs of all partials first, then the accumulators eight at a time
    float2 ml[kMaxSplit];
#pragma unroll
    for (int sp = 0; sp < kMaxSplit; ++sp)
      ml[sp] = sp < a.n_split ? *reinterpret_cast<const float2*>(a.part_ml + (first + sp * step) * 2) : make_float2(-INFINITY, 0.f);
    float M = -INFINITY;
#pragma unroll
    for (int sp = 0; sp < kMaxSplit; ++sp) M = fmaxf(M, ml[sp].x);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    float lsum = 0.f;
#pragma unroll
    for (int s0 = 0; s0 < kMaxSplit; s0 += 8) {
      if (s0 >= a.n_split) break;
      float4 p[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        p[u] = s0 + u < a.n_split ? *reinterpret_cast<const float4*>(a.part_acc + (first + (s0 + u) * step) * D + d)
                                  : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float m = ml[s0 + u].x;
        const float w = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - M);
        acc.x = fmaf(p[u].x, w, acc.x); acc.y = fmaf(p[u].y, w, acc.y); acc.z = fmaf(p[u].z, w, acc.z); acc.w = fmaf(p[u].w, w, acc.w);
        lsum = fmaf(ml[s0 + u].y, w, lsum);
      }
    }
    const float inv = 1.f / lsum;
    const bf16x4 ob = {(__bf16)(acc.x * inv), (__bf16)(acc.y * inv), (__bf16)(acc.z * inv), (__bf16)(acc.w * inv)};
    uint16_t* op = static_cast<uint16_t*>(a.o) + b * a.os_b + hq * a.os_h + (int64_t)(qtok - a.r_begin) * a.os_l + d;
    *reinterpret_cast<uint2*>(op) = __builtin_bit_cast(uint2, ob);
  }
}

// ---------------------------------------------------------------------------------------------------
// bf16 MFMA kernel for head dim 256.
//
// A wavefront's O accumulators (32 rows x 256 dims = 128 registers per lane) and Q fragments (64) leave no room for two
// wavefronts per SIMD, and four K + four V tiles of 32 KB do not fit the LDS: this kernel runs four wavefronts per
// workgroup, one per SIMD with the whole register file, over two K and two V tile buffers.  A wavefront owns 32 query
// rows of one q head (hpw q heads of the kv head x 4 / hpw blocks of 32 rows per workgroup); all walk the same key
// tiles: those whose largest row limit reaches the group's first query, found 64 tile summaries at a time with a
// ballot.  Fragment layouts, swizzles, lazy rescaling and the fused step (scores of tile j + 1 under the exponentials
// of tile j, then O += P V) are those of the kernel above.  With one wavefront per SIMD nothing else covers a wait, so
// the tile transfers are issued from assembly -- the compiler, which cannot tell the buffers apart, would otherwise
// wait for every transfer in flight before the first LDS read after it -- and the kernel orders them itself: a step
// begins with a wait for everything in flight and a workgroup barrier, requests K of tile j + 2 and V of tile j + 1,
// and reads K of tile j + 1 and V of tile j.  Chunks shorter than a tile are masked row by row (no packing).
// ---------------------------------------------------------------------------------------------------
struct WideSmem {
  uint16_t k[2][kTile * 256];  // K of tile j in k[j & 1]
  uint16_t v[2][kTile * 256];
  int limk[4][kTile];          // row limits of tile j in limk[j & 3]
};

// One global -> LDS transfer: lane i moves kBytes from its own global address to LDS address (uniform) + i * kBytes.
// Counted by vmcnt like any vector memory load.  (The host pass of the single-source compile never runs this.)
template <int kBytes>
__device__ __forceinline__ void lds_transfer(const void* gptr, const void* lds_ptr) {
#if defined(__HIP_DEVICE_COMPILE__)
  const uint32_t lds_addr =
      __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(const __attribute__((address_space(3))) unsigned char*)lds_ptr);
  if (kBytes == 16) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_addr) : "memory", "m0");
  } else {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(gptr), "s"(lds_addr) : "memory", "m0");
  }
#endif
}
// The LDS address of an object as a number: taken from the pointer once, it is plain scalar arithmetic from then on.
__device__ __forceinline__ uint32_t lds_address(const void* lds_ptr) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(const __attribute__((address_space(3))) unsigned char*)lds_ptr);
#else
  return 0;
#endif
}
// A 16-byte transfer with the global address as a uniform base (scalar registers) plus a byte offset per lane (no 64-bit
// vector arithmetic) and the LDS address as a number.
__device__ __forceinline__ void lds_transfer16_base(const void* base, uint32_t byte_off, uint32_t lds_addr) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(byte_off), "s"(base), "s"(lds_addr)
               : "memory", "m0");
#endif
}
__device__ __forceinline__ void wait_transfers() {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
}

constexpr int kWideWaves = 4;

__global__ __launch_bounds__(kWideWaves * kWave) void prefill_mfma_wide_kernel(PrefillArgs a) {
  constexpr int D = 256;
  constexpr int OCT = D / 8;
  constexpr int N_INST = kTile * OCT / kWave;        // 1 KiB transfers per tile
  constexpr int DMA_PER_WAVE = N_INST / kWideWaves;  // ... per wavefront and tensor
  constexpr int DSTEPS = D / 16;
  constexpr int DT = D / 32;
  constexpr int kHalf = kTile / 2;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  WideSmem& sm = *reinterpret_cast<WideSmem*>(smem_raw);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int hl = lane >> 5;

  int ks, hg, rank;
  map_workgroup(a, blockIdx.x, ks, hg, rank);
  const int qg = a.n_qg - 1 - rank;  // heavy query groups first
  const int b = ks / a.Hkv, hkv = ks % a.Hkv;
  const int hq = hkv * a.n_rep + hg * a.hpw + (wave % a.hpw);
  // (here qpw counts blocks of 32 query rows)
  const int blk_first = a.r_begin / kHalf, blk_last = (a.r_end - 1) / kHalf;
  const int blk_lo = blk_first + qg * a.qpw;
  const int blk_hi = min(blk_lo + a.qpw - 1, blk_last);
  const int my_blk = blk_lo + wave / a.hpw;
  const bool wave_live = my_blk <= blk_hi;
  const int q0 = my_blk * kHalf;  // region token of this wavefront's first row

  const int2* tl = a.tile_lim + (int64_t)ks * a.Tk;
  const int32_t* lim = a.tok_lim + (int64_t)ks * a.N;
  const uint16_t* kp = static_cast<const uint16_t*>(a.k) + b * a.ks_b + hkv * a.ks_h;
  const uint16_t* vp = static_cast<const uint16_t*>(a.v) + b * a.vs_b + hkv * a.vs_h;

  const int r0_group = max(blk_lo * kHalf, a.r_begin);
  const int rlast_group = min(blk_hi * kHalf + kHalf - 1, a.r_end - 1);
  const int my_r0 = max(q0, a.r_begin);
  const int my_rlast = min(q0 + kHalf - 1, a.r_end - 1);
  const int kt_end_group = (a.base + rlast_group) / kTile;

  // ---- Q fragments: B operand, lane (query l32, k-group hl) --------------------------------------
  bf16x8 qreg[DSTEPS];
  {
    const uint16_t* qp = static_cast<const uint16_t*>(a.q) + b * a.qs_b + hq * a.qs_h;
    int row = min(max(q0 + l32, a.r_begin), a.r_end - 1) - a.r_begin;
    const uint4* rp = reinterpret_cast<const uint4*>(qp + (int64_t)row * a.qs_l + hl * 8);
#pragma unroll
    for (int s = 0; s < DSTEPS; ++s) qreg[s] = __builtin_bit_cast(bf16x8, rp[s * 2]);
  }

  f32x16 oacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.f;
  float m_run = -INFINITY;
  float l_run = 0.f;
  const float c = a.scale * 1.4426950408889634f;

  // ---- the visited key tiles, in order: 64 summaries at a time (the same in every wavefront) --------
  int kt0 = 0;
  uint64_t vmask;
  int cmin;  // lane i: smallest row limit of tile kt0 + i
  auto refill = [&]() {
    const int t = kt0 + lane;
    const int2 val = tl[min(t, kt_end_group)];
    cmin = val.y;
    vmask = __ballot(t <= kt_end_group && val.x >= r0_group);
  };
  auto next_tile = [&](int& minlim) -> int {
    while (vmask == 0) {
      if (kt0 + kWave > kt_end_group) return -1;
      kt0 += kWave;
      refill();
    }
    const int i = __builtin_amdgcn_readfirstlane(__builtin_ctzll(vmask));
    vmask &= vmask - 1;
    minlim = __builtin_amdgcn_readlane(cmin, i);
    return kt0 + i;
  };
  refill();

  // ---- transfers ---------------------------------------------------------------------------------------
  auto v_swizzle = [](int row) { return (row & 3) << 2; };
  // Transfer j of this wavefront fills chunk slots [(wave * DMA_PER_WAVE + j) * 64, +64) of the LDS tile: rows
  // wave * 16 + 2 j + hl, chunk l32 of each.  The row part of the address is uniform (scalar arithmetic); the lane adds
  // hl rows and its swizzled chunk, which differs from transfer to transfer by an XOR with a constant: row % 32 =
  // (wave & 1) * 16 + 2 j + hl has its three parts in separate bits, and so has (row & 3) << 2 = (j & 1) << 3 | hl << 2.
  // Rows beyond N repeat row N-1 (they are later than every query, so the mask removes their scores).
  const uint32_t k_lane = (uint32_t)(hl * a.ks_l * 2), v_lane = (uint32_t)(hl * a.vs_l * 2);  // bytes
  const uint32_t k_chunk0 = (uint32_t)(l32 ^ (((wave & 1) << 4) | hl)), v_chunk0 = (uint32_t)(l32 ^ (hl << 2));
  const uint32_t lds_k0 = lds_address(&sm.k[0][0]), lds_v0 = lds_address(&sm.v[0][0]);
  auto issue_rows = [&](const uint16_t* base, int64_t stride, uint16_t* dst, int kt, bool is_v) {
    if (kt * kTile + kTile <= a.N) {
      const uint16_t* tb = base + ((int64_t)kt * kTile + wave * (2 * DMA_PER_WAVE)) * stride;  // uniform
      const uint32_t lds = (is_v ? lds_v0 + (uint32_t)((dst - &sm.v[0][0]) * 2) : lds_k0 + (uint32_t)((dst - &sm.k[0][0]) * 2)) +
                           (uint32_t)(wave * DMA_PER_WAVE * kWave * 16);
#pragma unroll
      for (int j = 0; j < DMA_PER_WAVE; ++j) {
        const uint32_t off = is_v ? v_lane + ((v_chunk0 ^ (uint32_t)((j & 1) << 3)) << 4) : k_lane + ((k_chunk0 ^ (uint32_t)(2 * j)) << 4);
        lds_transfer16_base(tb + (int64_t)(2 * j) * stride, off, lds + (uint32_t)(j * kWave * 16));
      }
    } else {
#pragma unroll
      for (int j = 0; j < DMA_PER_WAVE; ++j) {
        const int row = wave * (2 * DMA_PER_WAVE) + 2 * j + hl;
        const int chunk = is_v ? l32 ^ v_swizzle(row) : l32 ^ (row % OCT);
        const int n = min(kt * kTile + row, a.N - 1);
        lds_transfer<16>(base + (int64_t)n * stride + chunk * 8, dst + (wave * DMA_PER_WAVE + j) * kWave * 8);
      }
    }
  };
  auto issue_lim = [&](int kt, int slot) {
    if (wave == 0) lds_transfer<4>(lim + min(kt * kTile + lane, a.N - 1), &sm.limk[slot][0]);
  };
  auto issue_k = [&](int kt, int buf, int slot) {
    issue_rows(kp, a.ks_l, sm.k[buf], kt, false);
    issue_lim(kt, slot);
  };
  auto issue_v = [&](int kt, int buf) { issue_rows(vp, a.vs_l, sm.v[buf], kt, true); };

  // ---- operand fragments -------------------------------------------------------------------------------
  auto k_frag = [&](const uint16_t* Kt, int kb, int s) {
    const int row = kb * 32 + l32;
    const int chunk = (s * 2 + hl) ^ (row % OCT);
    return *reinterpret_cast<const bf16x8*>(Kt + row * D + chunk * 8);
  };
  const int r16 = lane & 15;
  const int dsel = (lane >> 4) & 1;
  auto v_frag = [&](const uint16_t* Vt, int t, int dt) {
    const int chunk0 = dt * 4 + dsel * 2 + ((r16 & 3) >> 1);
    const int half4 = (r16 & 1) * 4;
    const int row_lo = t * 16 + hl * 4 + (r16 >> 2);
    const int row_hi = row_lo + 8;
    const uint16_t* pl = Vt + row_lo * D + ((chunk0 ^ v_swizzle(row_lo)) * 8) + half4;
    const uint16_t* ph = Vt + row_hi * D + ((chunk0 ^ v_swizzle(row_hi)) * 8) + half4;
    bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4 __attribute__((address_space(3)))*)pl);
    bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4 __attribute__((address_space(3)))*)ph);
    bf16x8 va = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return va;
  };

  // scores of the first tile: nothing to run under, the K fragments are requested eight ahead
  auto qk_tile_first = [&](int buf, f32x16 (&sacc)[2]) {
    const uint16_t* Kt = sm.k[buf];
    constexpr int N_QK = 2 * DSTEPS;
    constexpr int AHEAD = 8;
    bf16x8 kf[AHEAD];
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) kf[i] = k_frag(Kt, i & 1, i >> 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < N_QK; ++i) {
      const int s = i >> 1, kb = i & 1;
      if (s == 0) {
        const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i % AHEAD], qreg[s], z, 0, 0, 0);
      } else {
        sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i % AHEAD], qreg[s], sacc[kb], 0, 0, 0);
      }
      if (i + AHEAD < N_QK) kf[i % AHEAD] = k_frag(Kt, (i + AHEAD) & 1, (i + AHEAD) >> 1);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto mask_scores = [&](int kt, int slot, f32x16 (&sv)[2]) {
    const int qtok = q0 + l32;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        int kk = kb * 32 + g4 * 8 + hl * 4;  // key offset in tile of accumulator 4*g4
        int4 lm = *reinterpret_cast<const int4*>(&sm.limk[slot][kk]);
        const int lv[4] = {lm.x, lm.y, lm.z, lm.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          int key = kt * kTile + kk + e - a.base;  // region token of the key row (negative: older row)
          bool vis = key <= qtok && qtok <= lv[e];
          if (!vis) sv[kb][g4 * 4 + e] = -INFINITY;
        }
      }
    }
  };
  auto row_max = [&](const f32x16 (&sv)[2]) {
    float m = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) m = fmaxf(m, sv[kb][i]);
    return half_swap_max(m) * c;
  };
  auto rescale = [&](float mx) {
    float m_new = fmaxf(m_run, mx);
    float alpha = m_run == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run - m_new);
    l_run *= alpha;
    m_run = m_new;
    // The accumulators live in the accumulation registers, which vector instructions reach only through moves.  The
    // moves are written here, in this rarely taken branch: left to the compiler, all 128 are read into vector
    // registers at the top of every step.  (The waits cover a matrix instruction that may still be writing.)
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float x = oacc[dt][i], tmp;
        asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\tv_accvgpr_write_b32 %0, %1"
                     : "+a"(x), "=&v"(tmp)
                     : "v"(alpha));
        oacc[dt][i] = x;
      }
    asm volatile("s_nop 4" ::: "memory");
#endif
  };
  // n-th probability of the tile in the order the PV MFMAs consume them (16 keys per B operand)
  auto prob = [&](const f32x16 (&sv)[2], int n, float m_use, float& rs, bf16x8 (&pb)[4]) {
    const int t = n >> 3, i = n & 7;
    float p = __builtin_amdgcn_exp2f(fmaf(sv[t >> 1][(t & 1) * 8 + i], c, -m_use));
    rs += p;
    pb[t][i] = (__bf16)p;
  };
  // scores of the next tile under the probabilities of keys 0..31 of this one, O += P V for keys 0..31 under the
  // probabilities of keys 32..63, then O += P V for keys 32..63; LDS operands are fetched two slots ahead
  auto fused_step = [&](int kbuf_next, int vbuf, const f32x16 (&sv)[2], f32x16 (&sacc)[2]) {
    const uint16_t* Kt = sm.k[kbuf_next];
    const uint16_t* Vt = sm.v[vbuf];
    constexpr int N_QK = 2 * DSTEPS;  // score MFMAs
    constexpr int N_PV = 4 * DT;      // PV MFMAs
    const float m_use = m_run == -INFINITY ? 0.f : m_run;
    float rs = 0.f;
    bf16x8 pb[4];
    int n = 0;
    __builtin_amdgcn_sched_barrier(0);
    auto k_at = [&](int i) { return k_frag(Kt, i & 1, i >> 1); };
    auto v_at = [&](int i) { return v_frag(Vt, i / DT, i % DT); };
    constexpr int R = 3;  // ring of operand fragments, fetched R - 1 slots ahead (deeper rings measure the same)
    bf16x8 kf[R], vf[R];
#pragma unroll
    for (int i = 0; i < R - 1; ++i) kf[i] = k_at(i);
#pragma unroll
    for (int i = 0; i < N_QK; ++i) {
      const int s = i >> 1, kb = i & 1;
      if (i + R - 1 < N_QK) {
        kf[(i + R - 1) % R] = k_at(i + R - 1);
      } else {
        vf[(i + R - 1 - N_QK) % R] = v_at(i + R - 1 - N_QK);
      }
      if (s == 0) {
        const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i % R], qreg[s], z, 0, 0, 0);
      } else {
        sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i % R], qreg[s], sacc[kb], 0, 0, 0);
      }
      if (n < 16) prob(sv, n++, m_use, rs, pb);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int i = 0; i < N_PV; ++i) {
      const int t = i / DT, dt = i % DT;
      if (i + R - 1 < N_PV) vf[(i + R - 1) % R] = v_at(i + R - 1);
      oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[i % R], pb[t], oacc[dt], 0, 0, 0);
      if (t < 2 && n < 32) prob(sv, n++, m_use, rs, pb);
      __builtin_amdgcn_sched_barrier(0);
    }
    l_run += rs;
  };

  // ---- tile loop -----------------------------------------------------------------------------------------
  int min_cur = 0, min_n1 = 0, min_n2 = 0;
  int t_cur = next_tile(min_cur);
  int t_n1 = t_cur >= 0 ? next_tile(min_n1) : -1;
  int t_n2 = t_n1 >= 0 ? next_tile(min_n2) : -1;
  f32x16 sacc[2];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int i = 0; i < 16; ++i) sacc[kb][i] = 0.f;
  if (t_cur >= 0) {
    issue_k(t_cur, 0, 0);
    issue_v(t_cur, 0);
    if (t_n1 >= 0) issue_k(t_n1, 1, 1);
    wait_transfers();
    __syncthreads();
    qk_tile_first(0, sacc);
  }
  for (int j = 0; t_cur >= 0; ++j) {
    // everything requested has landed, and every wavefront is through step j - 1: K of tile j and V of tile j - 1
    // have been read for the last time
    wait_transfers();
    __syncthreads();
    if (t_n2 >= 0) issue_k(t_n2, j & 1, (j + 2) & 3);
    if (t_n1 >= 0) issue_v(t_n1, (j + 1) & 1);
    f32x16 sv[2] = {sacc[0], sacc[1]};
    // no masked score: every key row is at or before the first query and visible to the last one
    const bool full = t_cur * kTile + kTile - 1 - a.base <= my_r0 && min_cur >= my_rlast;
    if (!full) mask_scores(t_cur, j & 3, sv);
    const float mx = row_max(sv);
    if (__builtin_expect(__ballot(mx > m_run + kRescaleSlack) != 0, 0)) rescale(mx);  // (rare: kept out of the way)
    fused_step((j + 1) & 1, j & 1, sv, sacc);  // (after the last tile: scores of a stale tile that nobody reads)
    t_cur = t_n1; min_cur = min_n1;
    t_n1 = t_n2; min_n1 = min_n2;
    t_n2 = t_n1 >= 0 ? next_tile(min_n2) : -1;
  }
  __syncthreads();  // the tile buffers are free

  // ---- epilogue: O rows go through LDS so that every row leaves as whole 16-byte pieces ----------------
  constexpr int kRowPitch = D * 2 + 16;  // bytes; the pad spreads the rows over the banks
  static_assert(kWideWaves * kHalf * kRowPitch <= sizeof(WideSmem), "staging area fits the tile buffers");
  unsigned char* stage = smem_raw + wave * (kHalf * kRowPitch);
  {
    const float l = half_swap_sum(l_run);
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        int d = dt * 32 + g4 * 8 + hl * 4;
        const bf16x4 ob = {(__bf16)(oacc[dt][g4 * 4 + 0] * inv), (__bf16)(oacc[dt][g4 * 4 + 1] * inv),
                           (__bf16)(oacc[dt][g4 * 4 + 2] * inv), (__bf16)(oacc[dt][g4 * 4 + 3] * inv)};
        *reinterpret_cast<uint2*>(stage + l32 * kRowPitch + d * 2) = __builtin_bit_cast(uint2, ob);
      }
    }
  }
  wave_lds_sync();
  if (wave_live) {
    uint16_t* op = static_cast<uint16_t*>(a.o) + b * a.os_b + hq * a.os_h;
    constexpr int kPieces = kHalf * OCT / kWave;  // 16-byte pieces per lane
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const int id = i * kWave + lane;
      const int row = id / OCT, piece = id % OCT;
      const int qtok = q0 + row;
      if (qtok >= a.r_begin && qtok < a.r_end) {
        const u32x4 val = *reinterpret_cast<const u32x4*>(stage + row * kRowPitch + piece * 16);
        __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(op + (int64_t)(qtok - a.r_begin) * a.os_l + piece * 8));
      }
    }
  }
}

static int launch_prefill_wide(const PrefillArgs& a, int64_t n_wg, hipStream_t st) {
  static bool configured[kMaxDevices] = {};  // the attribute is set once per device
  const size_t smem = sizeof(WideSmem);
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(NATS_ERR_LAUNCH, "prefill: no current device");
  if (!configured[dev]) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_mfma_wide_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return fail(NATS_ERR_LAUNCH, "hipFuncSetAttribute(%zu bytes of LDS): %s", smem, hipGetErrorString(e));
    configured[dev] = true;
  }
  hipLaunchKernelGGL(prefill_mfma_wide_kernel, dim3((unsigned)n_wg), dim3(kWideWaves * kWave), smem, st, a);
  NATS_CHECK_LAUNCH("prefill_mfma_wide_kernel");
  return NATS_OK;
}

template <int D, bool kUniform, int kMode = 0>
static int launch_prefill_mfma(const PrefillArgs& a, int64_t n_wg, hipStream_t st) {
  static bool configured[kMaxDevices] = {};  // per instantiation; the attribute is set once per device
  const size_t smem = sizeof(PrefillSmem<D>);
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(NATS_ERR_LAUNCH, "prefill: no current device");
  if (!configured[dev]) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_mfma_kernel<D, kUniform, kMode>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return fail(NATS_ERR_LAUNCH, "hipFuncSetAttribute(%zu bytes of LDS): %s", smem, hipGetErrorString(e));
    configured[dev] = true;
  }
  hipLaunchKernelGGL((prefill_mfma_kernel<D, kUniform, kMode>), dim3((unsigned)n_wg), dim3(kPrefillWaves * kWave), smem, st, a);
  NATS_CHECK_LAUNCH("prefill_mfma_kernel");
  return NATS_OK;
}

static int device_cu_count() {
  static int cached[kMaxDevices] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cached[dev] = n;
  }
  return cached[dev];
}

// Few query tiles over many key rows (a short segment over a long cache): how many workgroups share one tile list,
// so that the launch still fills the device.  1 = no split.
static bool use_split() {
  const char* e = getenv("NATS_PREFILL_SPLIT");
  return !(e && e[0] == '0');
}
static int choose_split(int64_t n_wg, int64_t Tk) {
  const int n_cu = device_cu_count();
  if (!use_split() || n_cu <= 0 || n_wg * 2 > n_cu) return 1;
  int64_t n = n_cu / n_wg;
  if (n > kMaxSplit) n = kMaxSplit;
  if (n > Tk / 4) n = Tk / 4;  // at least four key tiles per share
  return n < 2 ? 1 : (int)n;
}
static size_t split_partial_bytes(int64_t n_wg, int n_split, int64_t D) {
  return n_split <= 1 ? 0 : (size_t)n_wg * n_split * kPrefillWaves * (kTile / 2) * (D + 2) * sizeof(float);
}

}  // namespace nats

using namespace nats;

namespace {

struct SegmentShape {
  int64_t B, H_q, H_kv, D, C, W;
  int64_t x_len;    // queries
  int64_t N;        // key rows
  int64_t base;     // first key row of the open-chunk region
  int64_t r_begin;  // region token of query 0
};

int check_common(const char* who, const SegmentShape& g, const int64_t* q_strides, const int64_t* k_strides,
                 const int64_t* v_strides, const int64_t* o_strides, const void* q, const void* k, const void* v,
                 const void* o, int dtype) {
  NATS_REQUIRE(g.B > 0 && g.H_q > 0 && g.H_kv > 0 && g.x_len > 0, NATS_ERR_BAD_SHAPE, "%s: B=%lld H_q=%lld H_kv=%lld L=%lld",
               who, (long long)g.B, (long long)g.H_q, (long long)g.H_kv, (long long)g.x_len);
  NATS_REQUIRE(g.H_q % g.H_kv == 0, NATS_ERR_BAD_SHAPE, "%s: H_q=%lld is not a multiple of H_kv=%lld", who,
               (long long)g.H_q, (long long)g.H_kv);
  NATS_REQUIRE(g.D == 16 || g.D == 32 || g.D == 64 || g.D == 128 || g.D == 256, NATS_ERR_UNSUPPORTED,
               "%s: head_dim %lld (supported: 16, 32, 64, 128, 256)", who, (long long)g.D);
  NATS_REQUIRE(g.C > 0 && g.C < (int64_t(1) << 30), NATS_ERR_BAD_SHAPE, "%s: chunk size %lld", who, (long long)g.C);
  NATS_REQUIRE(g.W >= 0 && g.W % g.C == 0, NATS_ERR_BAD_SHAPE, "%s: window %lld is not a multiple of chunk size %lld", who,
               (long long)g.W, (long long)g.C);
  NATS_REQUIRE(dtype == NATS_DTYPE_BF16 || dtype == NATS_DTYPE_F32, NATS_ERR_BAD_DTYPE, "%s: dtype %d", who, dtype);
  NATS_REQUIRE(g.N < (int64_t(1) << 30), NATS_ERR_BAD_SHAPE, "%s: %lld key rows are too many", who, (long long)g.N);
  NATS_REQUIRE(k_strides[2] * kTile < (int64_t(1) << 30) && v_strides[2] * kTile < (int64_t(1) << 30) && k_strides[2] > 0 &&
                   v_strides[2] > 0,
               NATS_ERR_BAD_SHAPE, "%s: row strides %lld / %lld of k / v", who, (long long)k_strides[2], (long long)v_strides[2]);
  if (dtype == NATS_DTYPE_BF16 && (g.D == 32 || g.D == 64 || g.D == 128)) {
    // 16-byte vector loads and stores of rows
    NATS_REQUIRE(q_strides[2] % 8 == 0 && k_strides[2] % 8 == 0 && v_strides[2] % 8 == 0 && o_strides[2] % 8 == 0 &&
                     q_strides[1] % 8 == 0 && k_strides[1] % 8 == 0 && v_strides[1] % 8 == 0 && o_strides[1] % 8 == 0 &&
                     q_strides[0] % 8 == 0 && k_strides[0] % 8 == 0 && v_strides[0] % 8 == 0 && o_strides[0] % 8 == 0,
                 NATS_ERR_BAD_SHAPE, "%s: bf16 strides must keep rows 16-byte aligned", who);
    NATS_REQUIRE((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                  reinterpret_cast<uintptr_t>(o)) % 16 == 0,
                 NATS_ERR_BAD_SHAPE, "%s: bf16 tensors must be 16-byte aligned", who);
  }
  return NATS_OK;
}

bool use_packed_tiles() {
  const char* e = getenv("NATS_PREFILL_PACKED");
  return !(e && e[0] == '0');
}

bool use_far_rows() {
  const char* e = getenv("NATS_PREFILL_FAR");
  return !(e && e[0] == '0');
}

// key limits are in the workspace; launches the attention kernel of the segment
int launch_segment(const char* who, const SegmentShape& g, const void* q, const void* k, const void* v, void* o,
                   const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                   const int64_t* o_strides, float sm_scale, int dtype, const PrefillWorkspace& w, void* extra,
                   size_t extra_bytes, hipStream_t st) {
  PrefillArgs a{};
  a.q = q; a.k = k; a.v = v; a.o = o;
  a.tok_lim = w.tok_lim; a.tile_lim = w.tile_lim; a.gran_lim = w.gran_lim;
  a.qs_b = q_strides[0]; a.qs_h = q_strides[1]; a.qs_l = q_strides[2];
  a.ks_b = k_strides[0]; a.ks_h = k_strides[1]; a.ks_l = k_strides[2];
  a.vs_b = v_strides[0]; a.vs_h = v_strides[1]; a.vs_l = v_strides[2];
  a.os_b = o_strides[0]; a.os_h = o_strides[1]; a.os_l = o_strides[2];
  a.B = (int)g.B; a.Hq = (int)g.H_q; a.Hkv = (int)g.H_kv; a.n_rep = (int)(g.H_q / g.H_kv);
  a.N = (int)g.N; a.Tk = (int)((g.N + kTile - 1) / kTile);
  a.base = (int)g.base;
  a.r_begin = (int)g.r_begin; a.r_end = (int)(g.r_begin + g.x_len);
  a.qt_first = a.r_begin / kTile; a.qt_last = (a.r_end - 1) / kTile;
  const int64_t n_qt = a.qt_last - a.qt_first + 1;
  a.scale = sm_scale;
  a.hpw = 1; a.qpw = 1; a.n_hg = 1; a.n_qg = (int)n_qt; a.xcd_mode = 0;

  // bf16 at head dim 256 (rows that 16-byte transfers can take; other layouts go to the plain kernel)
  if (dtype == NATS_DTYPE_BF16 && g.D == 256) {
    bool rows16 = (reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                   reinterpret_cast<uintptr_t>(o)) % 16 == 0;
    for (int i = 0; i < 3; ++i)
      rows16 = rows16 && q_strides[i] % 8 == 0 && k_strides[i] % 8 == 0 && v_strides[i] % 8 == 0 && o_strides[i] % 8 == 0;
    if (rows16) {
      const int hpw = a.n_rep % 4 == 0 ? 4 : a.n_rep % 2 == 0 ? 2 : 1;
      a.hpw = hpw;
      a.qpw = kWideWaves / hpw;  // blocks of 32 query rows per workgroup
      a.n_hg = a.n_rep / hpw;
      const int64_t n_blk = (a.r_end - 1) / (kTile / 2) - a.r_begin / (kTile / 2) + 1;
      a.n_qg = (int)((n_blk + a.qpw - 1) / a.qpw);
      a.xcd_mode = ((g.B * g.H_kv) % 8 == 0) ? 1 : 0;
      a.n_split = 1;
      const int64_t n_wg = g.B * g.H_kv * a.n_hg * a.n_qg;
      NATS_REQUIRE(n_wg < (int64_t(1) << 31), NATS_ERR_BAD_SHAPE, "%s: grid too large", who);
      return launch_prefill_wide(a, n_wg, st);
    }
  }

  // fp32, and bf16 at the head dim the MFMA kernels do not take (16): the plain kernel
  if (dtype == NATS_DTYPE_F32 || (g.D != 32 && g.D != 64 && g.D != 128)) {
    NATS_REQUIRE(g.B * g.H_q <= 65535, NATS_ERR_BAD_SHAPE, "%s: B*H_q too large for the plain kernel", who);
    dim3 grid((unsigned)n_qt, (unsigned)(g.B * g.H_q));
    const bool f32 = dtype == NATS_DTYPE_F32;
#define NATS_PREFILL_PLAIN(DD)                                                                     \
  case DD:                                                                                         \
    if (f32) {                                                                                     \
      hipLaunchKernelGGL((prefill_simple_kernel<float, DD>), grid, dim3(64), 0, st, a);            \
    } else {                                                                                       \
      hipLaunchKernelGGL((prefill_simple_kernel<uint16_t, DD>), grid, dim3(64), 0, st, a);         \
    }                                                                                              \
    break;
    switch (g.D) {
      NATS_PREFILL_PLAIN(16)
      NATS_PREFILL_PLAIN(32)
      NATS_PREFILL_PLAIN(64)
      NATS_PREFILL_PLAIN(128)
      default:
      NATS_PREFILL_PLAIN(256)
    }
#undef NATS_PREFILL_PLAIN
    NATS_CHECK_LAUNCH("prefill_simple_kernel");
    return NATS_OK;
  }

  // bf16: pack the q heads of one kv head into one workgroup (up to 4), fill the rest with query tiles
  int n_rep = a.n_rep;
  int hpw = n_rep % 4 == 0 ? 4 : n_rep % 2 == 0 ? 2 : 1;  // (a group of 3, 5, 6, 7 ... goes in parts of 1 or 2 heads)
  a.hpw = hpw;
  a.qpw = 4 / hpw;
  a.n_hg = n_rep / hpw;
  a.n_qg = (int)((n_qt + a.qpw - 1) / a.qpw);
  a.xcd_mode = ((g.B * g.H_kv) % 8 == 0) ? 1 : 0;
  int64_t n_wg = g.B * g.H_kv * a.n_hg * a.n_qg;
  NATS_REQUIRE(n_wg < (int64_t(1) << 31), NATS_ERR_BAD_SHAPE, "%s: grid too large", who);
  // Packed tiles for chunks shorter than a tile, and for GQA groups of 1 and 2 at any chunk size: there the
  // workgroup's four or two query tiles walk one list together, which costs the same as every wavefront skipping
  // on its own between shared barriers and lets small launches share their lists among workgroups.
  const bool packed = (g.C < kTile || hpw < 4) && use_packed_tiles();
  // Chunks shorter than a granule: a granule far behind a query mostly holds a visible row or two among invisible
  // ones, so the rows more than a window (and a granule) behind a query group are taken from the lists of
  // long-lived rows instead, row by row (NATS_PREFILL_FAR=0 in the environment walks every granule, for comparison).
  // (Chunks of a granule and more: a visible granule is visible as a whole there, and its transfer from one base
  // address is cheaper than a gathered one; measured 10 % slower at chunk 32.)
  if (packed && g.C < kGranule && use_far_rows()) {
    a.t_long = (int)long_row_threshold(g.W);
    if (int rc = launch_long_rows(w, g.B * g.H_kv, g.N, g.base, g.W, st)) return rc;
    a.long_rows = w.long_rows; a.long_lim = w.long_lim; a.long_before = w.long_before; a.long_alive = w.long_alive;
    a.long_cap = (int)w.long_cap; a.n_gran = (int)w.n_gran; a.n_rtile = (int)w.n_rtile;
  }
  // (head dim -> instantiation)
#define NATS_PREFILL_BY_D(UNI, MODE, PA, NWG)                                                  \
  (g.D == 32 ? launch_prefill_mfma<32, UNI, MODE>(PA, NWG, st)                                 \
             : g.D == 64 ? launch_prefill_mfma<64, UNI, MODE>(PA, NWG, st) : launch_prefill_mfma<128, UNI, MODE>(PA, NWG, st))
  auto launch_packed = [&](const PrefillArgs& pa, int64_t n) {
    if (pa.long_rows) return NATS_PREFILL_BY_D(true, 2, pa, n);
    return NATS_PREFILL_BY_D(true, 1, pa, n);
  };
  a.n_split = 1;
  if (hpw == 4 || packed) {  // the kernels in which every wavefront walks the whole tile list
    const int ns = choose_split(n_wg, a.Tk);
    if (ns > 1 && extra && extra_bytes >= split_partial_bytes(n_wg, ns, g.D)) {
      a.n_split = ns;
      a.part_acc = static_cast<float*>(extra);
      a.part_ml = a.part_acc + (size_t)n_wg * ns * kPrefillWaves * (kTile / 2) * g.D;
    }
  }
  if (a.n_split > 1) {
    const int64_t n_launch = n_wg * a.n_split;
    int rc;
    if (packed) {
      rc = launch_packed(a, n_launch);
    } else {
      rc = NATS_PREFILL_BY_D(true, 0, a, n_launch);
    }
    if (rc) return rc;
    if (g.D == 32) {
      hipLaunchKernelGGL((prefill_split_merge_kernel<32>), dim3((unsigned)n_wg, kPrefillWaves * (kTile / 2) * 8 / 256), dim3(256), 0, st, a);
    } else if (g.D == 64) {
      hipLaunchKernelGGL((prefill_split_merge_kernel<64>), dim3((unsigned)n_wg, kPrefillWaves * (kTile / 2) * 16 / 256), dim3(256), 0, st, a);
    } else {
      hipLaunchKernelGGL((prefill_split_merge_kernel<128>), dim3((unsigned)n_wg, kPrefillWaves * (kTile / 2) * 32 / 256), dim3(256), 0, st, a);
    }
    NATS_CHECK_LAUNCH("prefill_split_merge_kernel");
    return NATS_OK;
  }
  // A launch of several rounds of workgroups per compute unit draws its lightest query groups from the counter
  // (NATS_PREFILL_POOL = eighths of the query groups that are drawn, 0 = none).
  {
    const char* e = getenv("NATS_PREFILL_POOL");
    const int eighths = e ? atoi(e) : 2;
    const int n_cu = device_cu_count();
    if (eighths > 0 && eighths <= 8 && w.ticket && n_cu > 0 && n_wg >= 4 * (int64_t)n_cu) {
      a.pool_ranks = (int)((int64_t)a.n_qg * eighths / 8);
      a.ticket = w.ticket;
      // the drawing workgroups loop: two per compute unit are enough (the grid stays a multiple of 8, XCD by XCD)
      const int64_t n_items = g.B * g.H_kv * a.n_hg;
      const int64_t pooled = n_items * a.pool_ranks;
      int64_t drawing = 2 * (int64_t)n_cu;
      if (drawing > pooled) drawing = pooled;
      n_wg = n_wg - pooled + (drawing + 7) / 8 * 8;
    }
  }
  // chunks shorter than a tile: tiles are packed from the 16-row granules that are visible (NATS_PREFILL_PACKED=0
  // in the environment keeps whole tiles, for comparison)
  // (GQA groups of 1 and 2: the workgroup's 2 or 4 query tiles form one group for the packing, every wavefront
  // walks the whole list and the element mask sorts out what its own rows see)
  if (packed)
    return launch_packed(a, n_wg);
  if (hpw == 4) return NATS_PREFILL_BY_D(true, 0, a, n_wg);
  return NATS_PREFILL_BY_D(false, 0, a, n_wg);
#undef NATS_PREFILL_BY_D
}

}  // namespace

extern "C" size_t nats_prefill_workspace_bytes(int64_t B, int64_t H_q, int64_t H_kv, int64_t L, int64_t D, int64_t C) {
  (void)D;
  if (B <= 0 || H_kv <= 0 || L <= 0 || C <= 0) return 0;
  return carve_prefill_workspace(nullptr, B * H_kv, (L + C - 1) / C, L).bytes + nats_prefill_sched_workspace_bytes(B, H_q, H_kv, L, L);
}

extern "C" size_t nats_prefill_sched_workspace_bytes(int64_t B, int64_t H_q, int64_t H_kv, int64_t n_queries, int64_t n_rows) {
  if (B <= 0 || H_q <= 0 || H_kv <= 0 || n_queries <= 0 || n_rows < n_queries) return 0;
  // a segment over a filled cache starts anywhere inside a 64-token tile of its region
  const int64_t n_qt = n_rows == n_queries ? (n_queries + kTile - 1) / kTile : (n_queries + kTile - 2) / kTile + 1;
  const int64_t Tk = (n_rows + kTile - 1) / kTile;
  const int64_t n_rep = H_q / H_kv;
  const int64_t hpw = n_rep % 4 == 0 ? 4 : n_rep % 2 == 0 ? 2 : 1;  // as in launch_segment
  // (a split launch never has more workgroups than the device has CUs, whatever the exact number of query tiles
  // turns out to be: room for that many partial results whenever a launch of this size may be split)
  const int64_t n_qg_min = (n_qt > 1 ? n_qt - 1 : 1) + 4 / hpw - 1;
  const int64_t n_wg_min = B * H_kv * (n_rep / hpw > 0 ? n_rep / hpw : 1) * (n_qg_min / (4 / hpw));
  return choose_split(n_wg_min, Tk) > 1 ? split_partial_bytes(device_cu_count(), 2, 128) / 2 : 0;
}

extern "C" size_t nats_prefill_past_workspace_bytes(int64_t B, int64_t H_kv, int64_t n_rows, int64_t S) {
  if (B <= 0 || H_kv <= 0 || n_rows <= 0 || S <= 0) return 0;
  return carve_prefill_workspace(nullptr, B * H_kv, S, n_rows).bytes;
}

extern "C" int nats_prefill_fwd(const void* q, const void* k, const void* v, const uint8_t* roles, void* o, int64_t B,
                                int64_t H_q, int64_t H_kv, int64_t L, int64_t D, int64_t C, int64_t W,
                                const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                const int64_t* o_strides, float sm_scale, int dtype, void* workspace,
                                size_t workspace_bytes, void* stream) {
  const char* who = "nats_prefill_fwd";
  NATS_REQUIRE(q && k && v && roles && o && workspace, NATS_ERR_NULL_POINTER, "%s: NULL pointer argument", who);
  NATS_REQUIRE(q_strides && k_strides && v_strides && o_strides, NATS_ERR_NULL_POINTER, "%s: NULL stride array", who);
  SegmentShape g{B, H_q, H_kv, D, C, W, L, L, 0, 0};
  if (int rc = check_common(who, g, q_strides, k_strides, v_strides, o_strides, q, k, v, o, dtype)) return rc;
  const int64_t S = (L + C - 1) / C;
  PrefillWorkspace w = carve_prefill_workspace(workspace, B * H_kv, S, L);
  NATS_REQUIRE(workspace_bytes >= w.bytes, NATS_ERR_WORKSPACE, "%s: workspace %zu bytes < %zu", who, workspace_bytes, w.bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (int rc = prepare_key_limits(roles, B, H_kv, S, L, C, W, nullptr, w, st)) return rc;
  return launch_segment(who, g, q, k, v, o, q_strides, k_strides, v_strides, o_strides, sm_scale, dtype, w,
                        static_cast<char*>(workspace) + w.bytes, workspace_bytes - w.bytes, st);
}

extern "C" int nats_prefill_past_fwd(const void* q, const void* cache_k, const void* cache_v, const uint8_t* valid,
                                     const int64_t* size_global, const int64_t* size_local, const uint8_t* roles, void* o,
                                     int64_t B, int64_t H_q, int64_t H_kv, int64_t x_len, int64_t D, int64_t C, int64_t W,
                                     const nats_past_state* state, const int64_t* q_strides, const int64_t* k_strides,
                                     const int64_t* v_strides, const int64_t* valid_strides, const int64_t* o_strides,
                                     float sm_scale, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  const char* who = "nats_prefill_past_fwd";
  NATS_REQUIRE(q && cache_k && cache_v && valid && size_global && size_local && roles && o && workspace,
               NATS_ERR_NULL_POINTER, "%s: NULL pointer argument", who);
  NATS_REQUIRE(q_strides && k_strides && v_strides && valid_strides && o_strides, NATS_ERR_NULL_POINTER,
               "%s: NULL stride array", who);
  NATS_REQUIRE(C > 0 && W >= 0 && W % C == 0, NATS_ERR_BAD_SHAPE, "%s: chunk size %lld, window %lld", who,
               (long long)C, (long long)W);
  if (int rc = check_past_state(who, state, x_len, C, W)) return rc;
  const int64_t base = state->n_ctx_data - state->old_fill;
  const int64_t N = state->n_ctx_data + x_len;
  SegmentShape g{B, H_q, H_kv, D, C, W, x_len, N, base, state->old_fill};
  if (int rc = check_common(who, g, q_strides, k_strides, v_strides, o_strides, q, cache_k, cache_v, o, dtype)) return rc;
  const int64_t S = (state->old_fill + x_len + C - 1) / C;
  PrefillWorkspace w = carve_prefill_workspace(workspace, B * H_kv, S, N);
  NATS_REQUIRE(workspace_bytes >= w.bytes, NATS_ERR_WORKSPACE, "%s: workspace %zu bytes < %zu", who, workspace_bytes, w.bytes);
  PastView pv{valid, valid_strides[0], valid_strides[1], size_global, size_local, base,
              state->gmin, state->tail, state->seen, state->fill_last, state->old_fill, state->update_chunk != 0};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (int rc = prepare_key_limits(roles, B, H_kv, S, N, C, W, &pv, w, st)) return rc;
  return launch_segment(who, g, q, cache_k, cache_v, o, q_strides, k_strides, v_strides, o_strides, sm_scale, dtype, w,
                        static_cast<char*>(workspace) + w.bytes, workspace_bytes - w.bytes, st);
}
