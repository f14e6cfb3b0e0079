// One-token decode attention over the evicted, ragged KV cache (HBM bound).
//
// Semantics: o[b, hq] = softmax over the rows i < n_rows with valid[b, hkv, i] != 0 of q . K[i] * scale, times V.
// (components/cache/nats_chunk_layer_cache.py:622-632 + SDPA; models/transformer/hf/llama.py:274-295.)
// Rows whose valid byte is 0 are never loaded, so whatever sits between a head's own end and the
// batch-wide n_ctx_data costs no bandwidth.
//
// Split-K: the rows of all (b, kv head) streams are cut into equal shares of 32-row tiles, one share per
// workgroup; inside a workgroup the four wavefronts take interleaved tiles, keep (m, l, acc) per q head and
// are merged through LDS; one partial per (workgroup, head touched) goes to the workspace and a second
// small kernel merges the partials of every q head.
#include <stdlib.h>

#include "nats_common.h"

#include <mutex>

namespace nats {

struct DecodeArgs {
  const void* q;
  const void* k;
  const void* v;
  const uint8_t* valid;
  const int64_t* row_end;  // optional [B*Hkv]: rows [row_end, tail_start) hold nothing valid and are skipped unseen
  void* o;
  float* ws_acc;  // [B*Hq, nsplit, D]
  float* ws_ml;   // [B*Hq, nsplit, 2]
  int64_t ks_b, ks_h, ks_r;
  int64_t vs_b, vs_h;
  int B, Hq, Hkv, n_rep;
  int n_rows, rows_per_split, nsplit;
  int tail_start;
  float scale;
  // balanced schedule of the bf16 kernel
  int2* head_table;  // [B*Hkv] {first partial slot, number of partials}
  int n_wg;          // workgroups along x
  int share_first;   // 1/256ths of the tiles that go to the first half of the workgroups (128: equal shares)
};

__device__ __forceinline__ float exp2_guard(float x) { return __builtin_amdgcn_exp2f(x); }

// ---------------------------------------------------------------------------------------------------
// bf16 kernel.  A wavefront walks 32-row tiles:
//   K rows go straight from global memory into the A operand of v_mfma_f32_16x16x32_bf16 (S^T = K Q^T, the
//   q heads of the group are the B columns, zero padded to 16);
//   V rows go global -> LDS without touching registers (global_load_lds, wave-private double buffer, 16-byte
//   chunks XOR-swizzled) and come back transposed through ds_read_b64_tr_b16 as the A operand of
//   O^T = V^T P^T; the probabilities are already in B-operand layout when they leave the softmax.
// Next tile's K (registers) and V (LDS) are requested before this tile's softmax and PV, so every
// wavefront keeps about 16 KiB in flight.  A row that is not valid is never read: its lane fetches the
// tile's first valid row instead (a cache hit), whose score is masked and whose probability is exactly 0.
// ---------------------------------------------------------------------------------------------------
constexpr float kDecodeRescaleSlack = 8.0f;
// K and V rows are read once per step: their loads carry the streaming hint (no retention in the caches)
constexpr int kAuxStream = 2;  // the "nt" bit of a global_load_lds
constexpr int kDecTile = 32;

constexpr int kMaxBalancedHeads = 1024;  // (b, kv head) streams whose tile prefix sums fit in LDS

template <int D, int NREP>
struct DecodeSmem {
  // [wave][buffer]; after a head's tile loop the wavefront's own buffers hold its accumulators
  // (NREP * D floats <= 2 * kDecTile * D bf16 for NREP <= 16)
  uint16_t v[4][2][kDecTile * D];
  float wm[4][NREP];
  float wl[4][NREP];
  int tile_prefix[kMaxBalancedHeads + 1];  // exclusive prefix of 32-row tiles per (b, kv head)
  int slot_prefix[kMaxBalancedHeads + 1];  // exclusive prefix of partial results per (b, kv head)
  int scan_tmp[256];
  int first_head;
};

// exclusive prefix sum over n <= kMaxBalancedHeads values held in `dst` (dst[n] receives the total)
__device__ __forceinline__ void block_exclusive_scan(int* dst, int n, int* tmp) {
  const int tid = threadIdx.x;
  const int per = (n + 255) / 256;
  const int lo = min(tid * per, n), hi = min(lo + per, n);
  int sum = 0;
  for (int i = lo; i < hi; ++i) sum += dst[i];
  tmp[tid] = sum;
  __syncthreads();
  if (tid < kWave) {  // wavefront 0 scans the 256 partial sums, 4 per lane
    int x0 = tmp[tid * 4], x1 = tmp[tid * 4 + 1], x2 = tmp[tid * 4 + 2], x3 = tmp[tid * 4 + 3];
    int mine = x0 + x1 + x2 + x3;
    int incl = mine;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      int y = __shfl_up(incl, o);
      if (tid >= o) incl += y;
    }
    int run = incl - mine;
    tmp[tid * 4] = run;
    tmp[tid * 4 + 1] = run + x0;
    tmp[tid * 4 + 2] = run + x0 + x1;
    tmp[tid * 4 + 3] = run + x0 + x1 + x2;
    if (tid == kWave - 1) dst[n] = incl;
  }
  __syncthreads();
  int run = tmp[tid];
  for (int i = lo; i < hi; ++i) {
    int x = dst[i];
    dst[i] = run;
    run += x;
  }
  __syncthreads();
}

// Balanced schedule: all 32-row tiles of all (b, kv head) streams form one list, cut into n_wg ranges (equal ones,
// or larger ones for the first half of the workgroups, see decode_share_first); a workgroup works through its
// range head by head and emits one partial (m, l, acc) per head it touches.  All finish together, whatever the
// per-head lengths are.
template <int D, int NREP>
__global__ __launch_bounds__(256) void decode_split_mfma_kernel(DecodeArgs a) {
  constexpr int STEPS = D / 32;      // k-steps of the score MFMA
  constexpr int OCT = D / 8;         // 16-byte chunks per row
  constexpr int NDMA = kDecTile * OCT / kWave;  // 1 KiB transfers per V tile
  constexpr int DB = D / 16;         // 16-dim blocks of O^T
  // V rows in LDS have their 16-byte chunks permuted so that the transposing reads of a half wavefront (four rows,
  // 32 bytes of each) spread over the banks; rows of 64 bytes only have four chunks to permute
  auto v_swz = [](int row) { return OCT >= 8 ? (row & 3) << 1 : (row >> 2) & 3; };

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  DecodeSmem<D, NREP>& sm = *reinterpret_cast<DecodeSmem<D, NREP>*>(smem_raw);

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int l16 = lane & 15;
  const int lg = lane >> 4;
  const int wg = blockIdx.x;
  const int grp = blockIdx.z;
  const int n_heads = a.B * a.Hkv;
  const int ts = a.row_end ? a.tail_start : a.n_rows;
  const int tail_tiles = (a.n_rows - ts + kDecTile - 1) / kDecTile;

  // ---- schedule: tiles per head, their prefix sums, this workgroup's range ----------------------------
  for (int h = tid; h < n_heads; h += 256) {
    int e = a.row_end ? (int)min((long long)a.row_end[h], (long long)ts) : a.n_rows;
    sm.tile_prefix[h] = (e + kDecTile - 1) / kDecTile + tail_tiles;
  }
  __syncthreads();
  block_exclusive_scan(sm.tile_prefix, n_heads, sm.scan_tmp);
  const int total = sm.tile_prefix[n_heads];
  // Tiles per workgroup: tpw_a for the first n_first workgroups (tiles [0, split)), tpw_b for the others.
  const int n_first = a.share_first == 128 ? a.n_wg : a.n_wg / 2;
  const int tpw_a = a.share_first == 128 ? (total + a.n_wg - 1) / a.n_wg
                                         : max(1, (int)(((int64_t)total * a.share_first / 256 + n_first - 1) / n_first));
  const int split = min(total, n_first * tpw_a);
  const int tpw_b = max(1, (total - split + (a.n_wg - n_first) - 1) / max(1, a.n_wg - n_first));
  auto wg_of = [&](int p) { return p < split ? p / tpw_a : n_first + (p - split) / tpw_b; };
  for (int h = tid; h < n_heads; h += 256) {
    int p0 = sm.tile_prefix[h], p1 = sm.tile_prefix[h + 1];
    sm.slot_prefix[h] = p1 > p0 ? wg_of(p1 - 1) - wg_of(p0) + 1 : 0;
  }
  __syncthreads();
  block_exclusive_scan(sm.slot_prefix, n_heads, sm.scan_tmp);
  if (wg == 0 && grp == 0) {
    for (int h = tid; h < n_heads; h += 256) {
      a.head_table[h] = make_int2(sm.slot_prefix[h], sm.slot_prefix[h + 1] - sm.slot_prefix[h]);
    }
  }
  int pos = wg < n_first ? wg * tpw_a : split + (wg - n_first) * tpw_b;
  const int pos_end = wg < n_first ? min(pos + tpw_a, split) : min(pos + tpw_b, total);
  if (pos >= pos_end) return;
  for (int h = tid; h < n_heads; h += 256) {
    if (sm.tile_prefix[h] <= pos && pos < sm.tile_prefix[h + 1]) sm.first_head = h;
  }
  __syncthreads();
  int ks = sm.first_head;  // b * Hkv + hkv
  const float c = a.scale * 1.4426950408889634f;

  const int nr = min(NREP, a.n_rep - grp * NREP);  // q heads of this group (the last group may hold fewer)

  // ---- state of the head being walked (set by begin_head) ----------------------------------------------
  const uint16_t* kp = nullptr;
  const uint16_t* vp = nullptr;
  const uint8_t* valp = nullptr;
  int e = 0, nA = 0;    // rows [0, e) and [ts, n_rows) are walked; nA = tiles of the first range
  int t = 0, t_end = 0; // this wavefront's next tile and the end of the workgroup's tiles, within the head
  int slot = 0;         // where the head's partial result goes
  int cur = 0;          // LDS buffer of tile t
  uint32_t vm = 0, vb_next = 0;
  bf16x8 qreg[STEPS];   // Q as the B operand: column = q head of the group (zero beyond nr), k = 8 dims per lane group
  uint4 kreg[2][STEPS];

  // Rows are walked in 32-row tiles over [0, e) and [ts, n_rows); [e, ts) is the dead region between this
  // head's own end and the open chunk (nothing there is valid), skipped without a look when hinted.
  auto tile_row0 = [&](int tt) -> int { return tt < nA ? tt * kDecTile : ts + (tt - nA) * kDecTile; };
  auto tile_row1 = [&](int tt) -> int {
    return tt < nA ? min(tt * kDecTile + kDecTile, e) : min(ts + (tt - nA + 1) * kDecTile, a.n_rows);
  };
  auto load_valid = [&](int tt) -> uint32_t {
    uint32_t vb = 0;
    if (tt < t_end) {
      int r0 = tile_row0(tt), r1 = tile_row1(tt);
      if (lane < kDecTile && r0 + lane < r1) vb = valp[r0 + lane];
    }
    return vb;
  };
  auto issue_k = [&](int r0, uint32_t m) {
    const int fv = __builtin_ctz(m);
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      int kl = g * 16 + l16;
      int row = ((m >> kl) & 1) ? kl : fv;
      const uint16_t* rp = kp + (int64_t)(r0 + row) * a.ks_r + lg * 8;
#pragma unroll
      for (int s = 0; s < STEPS; ++s) {
        const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(rp + s * 32));
        kreg[g][s] = make_uint4(w.x, w.y, w.z, w.w);
      }
    }
  };
  auto issue_v = [&](int r0, uint32_t m, int buf) {
    const int fv = __builtin_ctz(m);
#pragma unroll
    for (int j = 0; j < NDMA; ++j) {
      const int q = j * kWave + lane;  // chunk slot in the LDS tile
      const int row = q / OCT, cpos = q % OCT;
      const int src_row = ((m >> row) & 1) ? row : fv;
      const int chunk = cpos ^ v_swz(row);
      __builtin_amdgcn_global_load_lds(vp + (int64_t)(r0 + src_row) * a.ks_r + chunk * 8,
                                       (uint32_t __attribute__((address_space(3)))*)(&sm.v[wave][buf][j * kWave * 8]), 16, 0,
                                       kAuxStream);
    }
  };
  // Moves on to the head that holds tile `pos` of the list (`ks` is that head or an empty one before it): its
  // pointers and ranges, Q, and the requests for this wavefront's first tile, into LDS buffer `buf`.  Returns the
  // end of the workgroup's tiles in that head, as a list position.
  auto begin_head = [&](int buf) -> int {
    while (sm.tile_prefix[ks + 1] == sm.tile_prefix[ks]) ++ks;  // heads without tiles (pos < total: one with tiles follows)
    const int p0 = sm.tile_prefix[ks], p1 = sm.tile_prefix[ks + 1];
    const int seg_end = min(pos_end, p1);
    t_end = seg_end - p0;
    slot = sm.slot_prefix[ks] + (wg - wg_of(p0));
    const int b = ks / a.Hkv, hkv = ks % a.Hkv;
    const int hq0 = hkv * a.n_rep + grp * NREP;
    kp = static_cast<const uint16_t*>(a.k) + b * a.ks_b + hkv * a.ks_h;
    vp = static_cast<const uint16_t*>(a.v) + b * a.ks_b + hkv * a.ks_h;
    valp = a.valid + b * a.vs_b + hkv * a.vs_h;
    e = a.row_end ? (int)min((long long)a.row_end[ks], (long long)ts) : a.n_rows;
    nA = (e + kDecTile - 1) / kDecTile;
    const uint16_t* qp = static_cast<const uint16_t*>(a.q) + ((int64_t)b * a.Hq + hq0 + (l16 < nr ? l16 : 0)) * D;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      uint4 raw = *reinterpret_cast<const uint4*>(qp + s * 32 + lg * 8);
      if (l16 >= nr) raw = make_uint4(0, 0, 0, 0);
      qreg[s] = __builtin_bit_cast(bf16x8, raw);
    }
    t = pos - p0 + wave;
    cur = buf;
    vm = (uint32_t)__ballot(load_valid(t) != 0);
    if (vm) {
      issue_k(tile_row0(t), vm);
      issue_v(tile_row0(t), vm, cur);
    }
    vb_next = load_valid(t + 4);
    return seg_end;
  };

  int seg_end = begin_head(0);
  for (;;) {
    f32x4 oacc[DB];  // O^T block db: lane holds dims db*16 + lg*4 + i of q head l16
#pragma unroll
    for (int db = 0; db < DB; ++db) oacc[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;  // of q head l16 (meaningful for l16 < nr)

    while (t < t_end) {
      __builtin_amdgcn_s_waitcnt(0);  // K(t) in registers, V(t) in LDS, valid bytes of the next tile loaded
      const uint32_t vmn = (uint32_t)__ballot(vb_next != 0);
      float sc[2][4];
      float mx = -INFINITY;
      if (vm) {
        // scores: sc[g][i] belongs to key g*16 + lg*4 + i and q head l16
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < STEPS; ++s) {
            s4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kreg[g][s]), qreg[s], s4, 0, 0, 0);
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            int kl = g * 16 + lg * 4 + i;
            float sv = ((vm >> kl) & 1) ? s4[i] : -INFINITY;
            sc[g][i] = sv;
            mx = fmaxf(mx, sv);
          }
        }
      }
      // requests for the next tile go out before this tile's softmax and PV
      if (vmn) {
        issue_k(tile_row0(t + 4), vmn);
        issue_v(tile_row0(t + 4), vmn, cur ^ 1);
      }
      vb_next = load_valid(t + 8);

      if (vm) {
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32)) * c;  // vm != 0, so the maximum is finite
        // raise the running maximum only when it is exceeded by more than the slack (probabilities stay
        // below 2^slack otherwise); the accumulators are rescaled only then
        if (__ballot(l16 < nr && mx > m_run + kDecodeRescaleSlack)) {
          float m_new = fmaxf(m_run, mx);
          float alpha = m_run == -INFINITY ? 0.f : exp2_guard(m_run - m_new);
          l_run *= alpha;
          m_run = m_new;
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int i = 0; i < 4; ++i) oacc[db][i] *= alpha;
        }
        // P^T as the B operand: slot j < 4 is key lg*4 + j, slot j >= 4 is key 16 + lg*4 + (j - 4)
        bf16x8 pfrag;
        float rs = 0.f;
#pragma unroll
        for (int g = 0; g < 2; ++g) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float p = exp2_guard(fmaf(sc[g][i], c, -m_run));
            rs += p;
            pfrag[g * 4 + i] = (__bf16)p;
          }
        }
        l_run += rs;
        // V^T fragments: within 16 lanes, lane r reads 4 dims of key (K0 + r / 4) starting at dim
        // D0 + 4 * (r % 4) and receives keys K0 .. K0 + 3 of dim D0 + r (ds_read_b64_tr_b16)
        const uint16_t* Vt = sm.v[wave][cur];
        const int row_lo = lg * 4 + (l16 >> 2);
        const int row_hi = 16 + row_lo;
        const int half = l16 & 1;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const int chunk0 = db * 2 + ((l16 & 3) >> 1);
          const uint16_t* plo = Vt + row_lo * D + ((chunk0 ^ v_swz(row_lo)) * 8) + half * 4;
          const uint16_t* phi = Vt + row_hi * D + ((chunk0 ^ v_swz(row_hi)) * 8) + half * 4;
          bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4 __attribute__((address_space(3)))*)plo);
          bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4 __attribute__((address_space(3)))*)phi);
          bf16x8 va = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          oacc[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pfrag, oacc[db], 0, 0, 0);
        }
      }
      t += 4;
      vm = vmn;
      cur ^= 1;
    }
    __builtin_amdgcn_s_waitcnt(0);

    // ---- merge the wavefronts of the workgroup, emit this head's partial ------------------------------
    // The accumulators are staged in the wavefront's LDS buffer 0 (its tiles are consumed); the first tile of the
    // workgroup's next head, if there is one, is requested into buffer 1 before the merge, which hides most of its
    // trip from memory.
    l_run += __shfl_xor(l_run, 16);
    l_run += __shfl_xor(l_run, 32);
    float* wacc_mine = reinterpret_cast<float*>(&sm.v[wave][0][0]);  // [NREP][D]
    if (l16 < nr) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) wacc_mine[l16 * D + db * 16 + lg * 4 + i] = oacc[db][i];
    }
    if (lane < nr) {
      sm.wm[wave][lane] = m_run;
      sm.wl[wave][lane] = l_run;
    }
    const int slot_done = slot;
    pos = seg_end;
    const bool more = pos < pos_end;  // (the same for every wavefront of the workgroup)
    if (more) {
      ++ks;
      seg_end = begin_head(1);
    }
    __syncthreads();
    for (int idx = tid; idx < nr * D; idx += 256) {
      int h = idx / D, d = idx % D;
      float M = fmaxf(fmaxf(sm.wm[0][h], sm.wm[1][h]), fmaxf(sm.wm[2][h], sm.wm[3][h]));
      float sum = 0.f, lsum = 0.f;
      if (M != -INFINITY) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          float f = exp2_guard(sm.wm[w][h] - M);
          sum += reinterpret_cast<const float*>(&sm.v[w][0][0])[h * D + d] * f;
          lsum += sm.wl[w][h] * f;
        }
      }
      const int64_t prt = (int64_t)slot_done * a.n_rep + grp * NREP + h;  // partial of (slot, q head in the kv group)
      a.ws_acc[prt * D + d] = sum;
      if (d == 0) {
        a.ws_ml[prt * 2 + 0] = M;
        a.ws_ml[prt * 2 + 1] = lsum;
      }
    }
    if (!more) break;
    __syncthreads();  // the staged accumulators, wm and wl are reused by the next head
  }
}

// merge the partials of one q head (balanced schedule): grid = B*Hq, block = G * D threads (G groups of D threads).
// The weights 2^(m_s - M) of the partials are computed side by side (thread s takes partial s) and kept in LDS; group
// g then sums the accumulators of the partials g, g + G, ... in that order with four loads in flight, and the groups'
// sums are added in group order.  G = 1 for the few partials per head of a large batch; a single sequence, whose
// heads are cut among many workgroups, takes up to eight groups (the kernel is one trip to memory per four partials
// of a group, and nothing else).
constexpr int kMergeRed = 16;  // wavefronts of the largest block (1024 threads)
__global__ void decode_merge_balanced_kernel(const float* __restrict__ ws_acc, const float* __restrict__ ws_ml,
                                             const int2* __restrict__ head_table, uint16_t* __restrict__ o, int Hq, int Hkv,
                                             int D) {
  // [partials of the head] weights, 2 x kMergeRed floats for the block reductions, [G][D] sums of the groups
  extern __shared__ float merge_w[];
  const int head = blockIdx.x;  // b * Hq + hq
  const int tid = threadIdx.x;
  const int n_rep = Hq / Hkv;
  const int b = head / Hq, hq = head % Hq;
  const int2 tab = head_table[b * Hkv + hq / n_rep];
  const int r = hq % n_rep;
  const int n = tab.y;
  float* red = merge_w + n;
  float* part = red + 2 * kMergeRed;
  const int n_waves = (blockDim.x + kWave - 1) / kWave;

  float mloc = -INFINITY;
  for (int s = tid; s < n; s += blockDim.x) mloc = fmaxf(mloc, ws_ml[((int64_t)(tab.x + s) * n_rep + r) * 2]);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) mloc = fmaxf(mloc, __shfl_xor(mloc, off));
  if ((tid & 63) == 0) red[tid >> 6] = mloc;
  __syncthreads();
  float M = red[0];
  for (int w = 1; w < n_waves; ++w) M = fmaxf(M, red[w]);

  float lloc = 0.f;
  for (int s = tid; s < n; s += blockDim.x) {
    const int64_t prt = (int64_t)(tab.x + s) * n_rep + r;
    const float ms = ws_ml[prt * 2];
    const float f = (ms == -INFINITY) ? 0.f : exp2_guard(ms - M);
    merge_w[s] = f;
    lloc += ws_ml[prt * 2 + 1] * f;
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) lloc += __shfl_xor(lloc, off);
  if ((tid & 63) == 0) red[kMergeRed + (tid >> 6)] = lloc;
  __syncthreads();
  float lsum = red[kMergeRed];
  for (int w = 1; w < n_waves; ++w) lsum += red[kMergeRed + w];

  const int G = blockDim.x / D;
  const int g = tid / D, d = tid % D;
  float sum = 0.f;
  if (g < G) {
    const float* acc = ws_acc + ((int64_t)tab.x * n_rep + r) * D + d;
    const int64_t step = (int64_t)n_rep * D;
    int s = g;
    for (; s + 3 * G < n; s += 4 * G) {
      const float a0 = acc[s * step], a1 = acc[(s + G) * step], a2 = acc[(s + 2 * G) * step], a3 = acc[(s + 3 * G) * step];
      sum = fmaf(a0, merge_w[s], sum);
      sum = fmaf(a1, merge_w[s + G], sum);
      sum = fmaf(a2, merge_w[s + 2 * G], sum);
      sum = fmaf(a3, merge_w[s + 3 * G], sum);
    }
    for (; s < n; s += G) sum = fmaf(acc[s * step], merge_w[s], sum);
  }
  if (G > 1) {
    if (g < G) part[g * D + d] = sum;
    __syncthreads();
    if (g != 0) return;
    sum = part[d];
    for (int k = 1; k < G; ++k) sum += part[k * D + d];
  } else if (g != 0) {
    return;
  }
  o[(int64_t)head * D + d] = f32_to_bf16_bits(lsum > 0.f ? sum / lsum : 0.f);
}

// T = float, or uint16_t for bf16 at the head dim the MFMA kernel does not take (16).
template <typename T>
__device__ __forceinline__ float dec_load(const T* p);
template <>
__device__ __forceinline__ float dec_load<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float dec_load<uint16_t>(const uint16_t* p) { return bf16_bits_to_f32(*p); }

template <typename T, int D>
__global__ __launch_bounds__(256) void decode_split_f32_kernel(DecodeArgs a) {
  constexpr int LANES = D < 64 ? D : 64;  // lanes that hold dimensions of a row
  constexpr int PER = D / LANES;
  __shared__ float wacc[4][D];
  __shared__ float wm[4];
  __shared__ float wl[4];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int split = blockIdx.x;
  const int head = blockIdx.y;  // b * Hq + hq
  const int b = head / a.Hq, hq = head % a.Hq, hkv = hq / a.n_rep;
  const T* kp = static_cast<const T*>(a.k) + b * a.ks_b + hkv * a.ks_h;
  const T* vp = static_cast<const T*>(a.v) + b * a.ks_b + hkv * a.ks_h;
  const uint8_t* valp = a.valid + b * a.vs_b + hkv * a.vs_h;
  const T* qp = static_cast<const T*>(a.q) + (int64_t)head * D;
  const bool live = lane < LANES;
  const int d0 = live ? lane * PER : 0;
  float qv[PER], acc[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    qv[e] = live ? dec_load<T>(qp + d0 + e) : 0.f;
    acc[e] = 0.f;
  }
  float m_run = -INFINITY, l_run = 0.f;
  const int r_begin = split * a.rows_per_split;
  const int r_end = min(r_begin + a.rows_per_split, a.n_rows);
  for (int r = r_begin + wave; r < r_end; r += 4) {
    if (valp[r] == 0) continue;
    const T* kr = kp + (int64_t)r * a.ks_r;
    const T* vr = vp + (int64_t)r * a.ks_r;
    float dot = 0.f;
#pragma unroll
    for (int e = 0; e < PER; ++e) dot = fmaf(qv[e], dec_load<T>(kr + d0 + e), dot);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off);
    float s = dot * a.scale;
    float m_new = fmaxf(m_run, s);
    float alpha = expf(m_run - m_new);
    float p = expf(s - m_new);
    l_run = l_run * alpha + p;
#pragma unroll
    for (int e = 0; e < PER; ++e) acc[e] = fmaf(p, dec_load<T>(vr + d0 + e), acc[e] * alpha);
    m_run = m_new;
  }
  if (live) {
#pragma unroll
    for (int e = 0; e < PER; ++e) wacc[wave][d0 + e] = acc[e];
  }
  if (lane == 0) {
    wm[wave] = m_run;
    wl[wave] = l_run;
  }
  __syncthreads();
  for (int d = tid; d < D; d += 256) {
    float M = fmaxf(fmaxf(wm[0], wm[1]), fmaxf(wm[2], wm[3]));
    float sum = 0.f, lsum = 0.f;
    if (M != -INFINITY) {
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        float f = expf(wm[w] - M);
        sum += wacc[w][d] * f;
        lsum += wl[w] * f;
      }
    }
    a.ws_acc[((int64_t)head * a.nsplit + split) * D + d] = sum;
    if (d == 0) {
      // the merge kernel works in the base-2 domain
      a.ws_ml[((int64_t)head * a.nsplit + split) * 2 + 0] = M == -INFINITY ? M : M * 1.4426950408889634f;
      a.ws_ml[((int64_t)head * a.nsplit + split) * 2 + 1] = lsum;
    }
  }
}

// merge the splits of one q head: grid = B*Hq, block = D threads
template <bool kBf16Out>
__global__ void decode_merge_kernel(const float* __restrict__ ws_acc, const float* __restrict__ ws_ml, void* __restrict__ o,
                                    int nsplit, int D) {
  const int head = blockIdx.x;
  const int d = threadIdx.x;
  if (d >= D) return;
  const float* ml = ws_ml + (int64_t)head * nsplit * 2;
  float M = -INFINITY;
  for (int s = 0; s < nsplit; ++s) M = fmaxf(M, ml[2 * s]);
  float sum = 0.f, lsum = 0.f;
  if (M != -INFINITY) {
    for (int s = 0; s < nsplit; ++s) {
      float ms = ml[2 * s];
      if (ms == -INFINITY) continue;
      float f = exp2_guard(ms - M);
      sum += ws_acc[((int64_t)head * nsplit + s) * D + d] * f;
      lsum += ml[2 * s + 1] * f;
    }
  }
  float out = lsum > 0.f ? sum / lsum : 0.f;
  if (kBf16Out) {
    static_cast<uint16_t*>(o)[(int64_t)head * D + d] = f32_to_bf16_bits(out);
  } else {
    static_cast<float*>(o)[(int64_t)head * D + d] = out;
  }
}

static void decode_split_geometry(int64_t B, int64_t H_kv, int64_t n_rows, int* rows_per_split, int* nsplit) {
  int64_t streams = B * H_kv;
  int64_t want = 2048 / (streams > 0 ? streams : 1);
  if (want < 1) want = 1;
  int64_t r = (n_rows + want - 1) / want;
  r = ((r + 255) / 256) * 256;
  if (r < 256) r = 256;
  if (r > 8192) r = 8192;
  *rows_per_split = (int)r;
  // the walk over [0, row_end) and [tail_start, n_rows) can take one 32-row tile more than ceil(n_rows / 32)
  *nsplit = (int)((n_rows + 32 + r - 1) / r);
}

static int compute_units_of_current_device() {
  static int n_cu_of[64] = {};  // compute units of every device, asked for once each
  int dev = 0, n_cu = 256;
  if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64) {
    if (n_cu_of[dev] == 0) {
      int v = 0;
      n_cu_of[dev] = (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) ? v : 256;
    }
    n_cu = n_cu_of[dev];
  }
  return n_cu;
}

// workgroups of the balanced bf16 schedule: two per compute unit, fewer when there is little to do
static int decode_balanced_workgroups(int64_t B, int64_t H_kv, int64_t n_rows) {
  int64_t upper = B * H_kv * ((n_rows + kDecTile - 1) / kDecTile + 1);  // tiles, at most
  int64_t want = (upper + 7) / 8;                                        // at least 8 tiles per workgroup
  int64_t cap = 2 * (int64_t)compute_units_of_current_device();
  return (int)(want < 1 ? 1 : (want > cap ? cap : want));
}

// Share of the tiles that the first half of the workgroups takes, in 1/256ths.  When the grid is exactly two
// workgroups per compute unit, the first half of the grid is every unit's first resident workgroup, and that one
// is served about twice as fast as the second while both are resident (measured with device timestamps: with equal
// shares the first halves end after 210 us of a 285 us launch and the units then run half empty).  With 176/256 of
// the tiles on the first half both halves end together.  NATS_DECODE_SHARE overrides the share (128: equal).
static int decode_share_first(int n_wg, int groups) {
  if (n_wg < 2 || n_wg % 2 != 0) return 128;
  const char* e = getenv("NATS_DECODE_SHARE");
  if (e) {
    const int v = atoi(e);
    return v > 0 && v < 256 ? v : 128;
  }
  return (groups == 1 && n_wg == 2 * compute_units_of_current_device()) ? 176 : 128;
}

static size_t align256(size_t x) { return (x + 255) & ~size_t(255); }

template <int D, int NREP>
static int launch_mfma(const DecodeArgs& a, int groups, hipStream_t st) {
  static bool configured[64] = {};  // per instantiation; the LDS attribute is set once per device
  const size_t smem = sizeof(DecodeSmem<D, NREP>);
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fail(NATS_ERR_LAUNCH, "decode: no current device");
  if (!configured[dev]) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&decode_split_mfma_kernel<D, NREP>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return fail(NATS_ERR_LAUNCH, "hipFuncSetAttribute(%zu bytes of LDS): %s", smem, hipGetErrorString(e));
    configured[dev] = true;
  }
  dim3 grid((unsigned)a.n_wg, 1u, (unsigned)groups);
  hipLaunchKernelGGL((decode_split_mfma_kernel<D, NREP>), grid, dim3(256), smem, st, a);
  return NATS_OK;
}

}  // namespace nats

using namespace nats;

extern "C" size_t nats_decode_workspace_bytes(int64_t B, int64_t H_q, int64_t H_kv, int64_t D, int64_t n_rows) {
  if (B <= 0 || H_q <= 0 || H_kv <= 0 || D <= 0 || n_rows <= 0) return 0;
  int rps, ns;
  decode_split_geometry(B, H_kv, n_rows, &rps, &ns);
  size_t split_layout = (size_t)B * H_q * ns * (D + 2) * sizeof(float);  // fp32 kernel: [q head][split]
  size_t slots = (size_t)decode_balanced_workgroups(B, H_kv, n_rows) + (size_t)(B * H_kv);
  size_t balanced_layout = align256((size_t)(B * H_kv) * sizeof(int2)) + slots * (H_q / H_kv) * (D + 2) * sizeof(float);
  return split_layout > balanced_layout ? split_layout : balanced_layout;
}

// `workspace` is caller memory (nats_decode_fwd) or the library's static scratch array (nats_decode_fwd_static);
// `max_bytes` != 0 names the fixed size of the latter, for the error text.
static int decode_fwd_impl(const void* q, const void* cache_k, const void* cache_v, const uint8_t* valid,
                           const int64_t* row_end, int64_t tail_start, void* o, int64_t B, int64_t H_q, int64_t H_kv,
                           int64_t D, int64_t n_rows, const int64_t* kv_strides, const int64_t* valid_strides,
                           float sm_scale, int dtype, void* workspace, size_t workspace_bytes, size_t max_bytes,
                           void* stream) {
  NATS_REQUIRE(q && cache_k && cache_v && valid && o && workspace, NATS_ERR_NULL_POINTER,
               "nats_decode_fwd: NULL pointer argument");
  NATS_REQUIRE(kv_strides && valid_strides, NATS_ERR_NULL_POINTER, "nats_decode_fwd: NULL stride array");
  NATS_REQUIRE(B > 0 && H_q > 0 && H_kv > 0 && n_rows > 0, NATS_ERR_BAD_SHAPE,
               "nats_decode_fwd: B=%lld H_q=%lld H_kv=%lld n_rows=%lld", (long long)B, (long long)H_q, (long long)H_kv,
               (long long)n_rows);
  NATS_REQUIRE(H_q % H_kv == 0, NATS_ERR_BAD_SHAPE, "nats_decode_fwd: H_q=%lld is not a multiple of H_kv=%lld",
               (long long)H_q, (long long)H_kv);
  NATS_REQUIRE(D == 16 || D == 32 || D == 64 || D == 128 || D == 256, NATS_ERR_UNSUPPORTED,
               "nats_decode_fwd: head_dim %lld (supported: 16, 32, 64, 128, 256)", (long long)D);
  const bool mfma = dtype == NATS_DTYPE_BF16 && D >= 32;  // bf16 at head dim 16 takes the plain kernel
  NATS_REQUIRE(dtype == NATS_DTYPE_BF16 || dtype == NATS_DTYPE_F32, NATS_ERR_BAD_DTYPE, "nats_decode_fwd: dtype %d", dtype);
  NATS_REQUIRE(n_rows < (int64_t(1) << 30) && B * H_q <= (int64_t(1) << 30), NATS_ERR_BAD_SHAPE,
               "nats_decode_fwd: problem too large");
  NATS_REQUIRE(B * H_kv <= 65535 && B * H_q <= 65535 * 16, NATS_ERR_BAD_SHAPE, "nats_decode_fwd: too many (b, head) streams");
  NATS_REQUIRE(row_end == nullptr || (tail_start >= 0 && tail_start <= n_rows), NATS_ERR_BAD_SHAPE,
               "nats_decode_fwd: tail_start=%lld outside [0, n_rows=%lld]", (long long)tail_start, (long long)n_rows);
  size_t need = nats_decode_workspace_bytes(B, H_q, H_kv, D, n_rows);
  NATS_REQUIRE(max_bytes == 0 || need <= max_bytes, NATS_ERR_WORKSPACE,
               "nats_decode_fwd_static: this shape needs %zu bytes of scratch, the static array holds %zu; use "
               "nats_decode_fwd with a caller workspace",
               need, max_bytes);
  NATS_REQUIRE(workspace_bytes >= need, NATS_ERR_WORKSPACE, "nats_decode_fwd: workspace %zu bytes < %zu", workspace_bytes,
               need);
  if (mfma) {
    NATS_REQUIRE(kv_strides[0] % 8 == 0 && kv_strides[1] % 8 == 0 && kv_strides[2] % 8 == 0, NATS_ERR_BAD_SHAPE,
                 "nats_decode_fwd: bf16 cache strides must keep rows 16-byte aligned");
    NATS_REQUIRE((reinterpret_cast<uintptr_t>(cache_k) | reinterpret_cast<uintptr_t>(cache_v) |
                  reinterpret_cast<uintptr_t>(q)) % 16 == 0,
                 NATS_ERR_BAD_SHAPE, "nats_decode_fwd: bf16 tensors must be 16-byte aligned");
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  DecodeArgs a;
  a.q = q; a.k = cache_k; a.v = cache_v; a.valid = valid; a.o = o;
  a.row_end = mfma ? row_end : nullptr;
  a.tail_start = (int)tail_start;
  a.ks_b = kv_strides[0]; a.ks_h = kv_strides[1]; a.ks_r = kv_strides[2];
  a.vs_b = valid_strides[0]; a.vs_h = valid_strides[1];
  a.B = (int)B; a.Hq = (int)H_q; a.Hkv = (int)H_kv; a.n_rep = (int)(H_q / H_kv);
  a.n_rows = (int)n_rows;
  decode_split_geometry(B, H_kv, n_rows, &a.rows_per_split, &a.nsplit);
  a.scale = sm_scale;
  a.head_table = nullptr;
  a.n_wg = 0;
  a.share_first = 128;
  a.ws_acc = static_cast<float*>(workspace);
  a.ws_ml = a.ws_acc + (size_t)B * H_q * a.nsplit * D;

  if (!mfma) {
    dim3 grid((unsigned)a.nsplit, (unsigned)(B * H_q));
    const bool f32 = dtype == NATS_DTYPE_F32;
#define NATS_DECODE_PLAIN(DD)                                                                        \
  case DD:                                                                                           \
    if (f32) {                                                                                       \
      hipLaunchKernelGGL((decode_split_f32_kernel<float, DD>), grid, dim3(256), 0, st, a);           \
    } else {                                                                                         \
      hipLaunchKernelGGL((decode_split_f32_kernel<uint16_t, DD>), grid, dim3(256), 0, st, a);        \
    }                                                                                                \
    break;
    switch (D) {
      NATS_DECODE_PLAIN(16)
      NATS_DECODE_PLAIN(32)
      NATS_DECODE_PLAIN(64)
      NATS_DECODE_PLAIN(128)
      default:
      NATS_DECODE_PLAIN(256)
    }
#undef NATS_DECODE_PLAIN
    NATS_CHECK_LAUNCH("decode_split_f32_kernel");
    if (f32) {
      hipLaunchKernelGGL((decode_merge_kernel<false>), dim3((unsigned)(B * H_q)), dim3((unsigned)D), 0, st, a.ws_acc, a.ws_ml,
                         o, a.nsplit, (int)D);
    } else {
      hipLaunchKernelGGL((decode_merge_kernel<true>), dim3((unsigned)(B * H_q)), dim3((unsigned)D), 0, st, a.ws_acc, a.ws_ml,
                         o, a.nsplit, (int)D);
    }
    NATS_CHECK_LAUNCH("decode_merge_kernel");
    return NATS_OK;
  }

  NATS_REQUIRE(H_kv <= kMaxBalancedHeads, NATS_ERR_UNSUPPORTED,
               "nats_decode_fwd: %lld kv heads, the bf16 kernel schedules at most %d per sequence", (long long)H_kv,
               kMaxBalancedHeads);
  // One launch pair schedules at most kMaxBalancedHeads (b, kv head) streams (their prefix sums live in LDS); a
  // larger batch goes in groups of whole sequences, one after the other on the stream, over the same workspace.
  const int64_t b_step = kMaxBalancedHeads / H_kv;
  const int n_rep = a.n_rep;
  // q heads of a kv head share the key / value rows of one pass, up to eight at a time (columns of the MFMA);
  // a group size that is no power of two runs the next wider kernel with its spare columns zero
  const int nrep_k = n_rep >= 5 ? 8 : n_rep >= 3 ? 4 : n_rep;
  const int groups = (n_rep + nrep_k - 1) / nrep_k;
  for (int64_t b0 = 0; b0 < B; b0 += b_step) {
    const int64_t nb = B - b0 < b_step ? B - b0 : b_step;
    DecodeArgs c = a;
    c.B = (int)nb;
    c.q = static_cast<const uint16_t*>(q) + b0 * H_q * D;
    c.k = static_cast<const uint16_t*>(cache_k) + b0 * a.ks_b;
    c.v = static_cast<const uint16_t*>(cache_v) + b0 * a.ks_b;
    c.valid = valid + b0 * a.vs_b;
    c.row_end = a.row_end ? a.row_end + b0 * H_kv : nullptr;
    c.o = static_cast<uint16_t*>(o) + b0 * H_q * D;
    c.n_wg = decode_balanced_workgroups(nb, H_kv, n_rows);
    // (rows of 512 bytes: a workgroup's V buffers take 128 KB of LDS, so one workgroup fits a compute unit at a time; one
    // round of workgroups with equal shares measures 1 % faster than two)
    if (D == 256) c.n_wg = std::min(c.n_wg, compute_units_of_current_device());
    c.share_first = decode_share_first(c.n_wg, groups);
    c.head_table = static_cast<int2*>(workspace);
    c.ws_acc = reinterpret_cast<float*>(static_cast<char*>(workspace) + align256((size_t)(nb * H_kv) * sizeof(int2)));
    c.ws_ml = c.ws_acc + ((size_t)c.n_wg + (size_t)(nb * H_kv)) * (size_t)n_rep * D;
    int rc;
    if (D == 128) {
      switch (nrep_k) {
        case 8: rc = launch_mfma<128, 8>(c, groups, st); break;
        case 4: rc = launch_mfma<128, 4>(c, groups, st); break;
        case 2: rc = launch_mfma<128, 2>(c, groups, st); break;
        default: rc = launch_mfma<128, 1>(c, groups, st); break;
      }
    } else if (D == 256) {
      c.share_first = 128;
      switch (nrep_k) {
        case 8: rc = launch_mfma<256, 8>(c, groups, st); break;
        case 4: rc = launch_mfma<256, 4>(c, groups, st); break;
        case 2: rc = launch_mfma<256, 2>(c, groups, st); break;
        default: rc = launch_mfma<256, 1>(c, groups, st); break;
      }
    } else if (D == 32) {
      switch (nrep_k) {
        case 8: rc = launch_mfma<32, 8>(c, groups, st); break;
        case 4: rc = launch_mfma<32, 4>(c, groups, st); break;
        case 2: rc = launch_mfma<32, 2>(c, groups, st); break;
        default: rc = launch_mfma<32, 1>(c, groups, st); break;
      }
    } else {
      switch (nrep_k) {
        case 8: rc = launch_mfma<64, 8>(c, groups, st); break;
        case 4: rc = launch_mfma<64, 4>(c, groups, st); break;
        case 2: rc = launch_mfma<64, 2>(c, groups, st); break;
        default: rc = launch_mfma<64, 1>(c, groups, st); break;
      }
    }
    if (rc) return rc;
    NATS_CHECK_LAUNCH("decode_split_mfma_kernel");
    // (a head has at most one partial per workgroup plus one)
    // groups of the merge kernel's block: about four partials per group and head
    const int64_t per_head = c.n_wg / (nb * H_kv) + 1;
    int merge_groups = 1;
    while (merge_groups < 8 && merge_groups * 4 < per_head && (merge_groups * 2) * D <= 1024) merge_groups *= 2;
    const size_t merge_smem = ((size_t)c.n_wg + 2 + 2 * kMergeRed + (size_t)merge_groups * D) * sizeof(float);
    hipLaunchKernelGGL(decode_merge_balanced_kernel, dim3((unsigned)(nb * H_q)), dim3((unsigned)(merge_groups * D)), merge_smem, st, c.ws_acc,
                       c.ws_ml, c.head_table, static_cast<uint16_t*>(c.o), (int)H_q, (int)H_kv, (int)D);
    NATS_CHECK_LAUNCH("decode_merge_balanced_kernel");
  }
  return NATS_OK;
}

extern "C" int nats_decode_fwd(const void* q, const void* cache_k, const void* cache_v, const uint8_t* valid,
                               const int64_t* row_end, int64_t tail_start, void* o, int64_t B, int64_t H_q, int64_t H_kv,
                               int64_t D, int64_t n_rows, const int64_t* kv_strides, const int64_t* valid_strides,
                               float sm_scale, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  return decode_fwd_impl(q, cache_k, cache_v, valid, row_end, tail_start, o, B, H_q, H_kv, D, n_rows, kv_strides,
                         valid_strides, sm_scale, dtype, workspace, workspace_bytes, 0, stream);
}

// ---------------------------------------------------------------------------------------------------
// The same op for callers that cannot allocate: the partial results live in a static device array.
// ---------------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[NATS_DECODE_STATIC_SCRATCH_BYTES];

// Every device holds its own copy of `scratch` at its own address; in host code the array's name is only a
// handle for hipGetSymbolAddress, never a device address.  Looked up once per device, with that device current.
static int static_scratch_of_current_device(void** out) {
  static std::mutex mu;
  static void* ptr_of[64] = {};
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= 64)
    return fail(NATS_ERR_LAUNCH, "nats_decode_fwd_static: no current device (%s)", hipGetErrorString(e));
  std::lock_guard<std::mutex> lock(mu);
  if (ptr_of[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return fail(NATS_ERR_LAUNCH, "nats_decode_fwd_static: hipGetSymbolAddress(scratch) on device %d: %s", dev,
                  hipGetErrorString(e));
    ptr_of[dev] = p;
  }
  *out = ptr_of[dev];
  return NATS_OK;
}

extern "C" size_t nats_decode_static_scratch_bytes(void) { return NATS_DECODE_STATIC_SCRATCH_BYTES; }

extern "C" int nats_decode_fwd_static(const void* q, const void* cache_k, const void* cache_v, const uint8_t* valid,
                                      const int64_t* row_end, int64_t tail_start, void* o, int64_t B, int64_t H_q,
                                      int64_t H_kv, int64_t D, int64_t n_rows, const int64_t* kv_strides,
                                      const int64_t* valid_strides, float sm_scale, int dtype, void* stream) {
  void* ws = nullptr;
  if (int rc = static_scratch_of_current_device(&ws)) return rc;
  // Nothing in the scratch has to start at zero: the split kernels write every partial sum, maximum, row sum and
  // head-table entry that the merge kernels of the same call read.
  return decode_fwd_impl(q, cache_k, cache_v, valid, row_end, tail_start, o, B, H_q, H_kv, D, n_rows, kv_strides,
                         valid_strides, sm_scale, dtype, ws, NATS_DECODE_STATIC_SCRATCH_BYTES,
                         NATS_DECODE_STATIC_SCRATCH_BYTES, stream);
}
