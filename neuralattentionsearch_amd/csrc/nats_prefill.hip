// Role-masked, chunked flash-attention prefill for gfx950.
//
// Two kernels share one tile-skip map:
//   prefill_mfma_kernel   bf16, QK^T and PV on v_mfma_f32_32x32x16_bf16, fp32 online softmax
//   prefill_simple_kernel fp32 (or bf16) FMA kernel, one query row per lane; the fp32 parity path
//
// Mask semantics (components/masks/utils.py:89-94, components/cache/nats_chunk_layer_cache.py:603-616):
// query token m sees key token n iff n <= m and slot(m) <= vis_lim[slot(n)].
#include "nats_common.h"

namespace nats {

int launch_role_scan(const uint8_t* roles, int64_t n_streams, int64_t S, int64_t W, int64_t C, int64_t* end_idx,
                     int32_t* vis_lim, hipStream_t st);
int launch_tile_lim(const int32_t* vis_lim, int64_t n_streams, int64_t S, int64_t T, int64_t C, int2* tile_lim,
                    hipStream_t st);

struct PrefillArgs {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  const int32_t* vis_lim;  // [B*Hkv, S]
  const int2* tile_lim;    // [B*Hkv, T] {max, min}
  int64_t qs_b, qs_h, qs_l;
  int64_t ks_b, ks_h, ks_l;
  int64_t vs_b, vs_h, vs_l;
  int64_t os_b, os_h, os_l;
  int B, Hq, Hkv, n_rep;
  int L, S, T;
  int c_shift;
  int hpw;       // q heads of one kv head handled by one workgroup (mfma kernel)
  int qpw;       // 64-row query tiles handled by one workgroup (mfma kernel)
  int n_hg;      // head groups per kv head = n_rep / hpw
  int n_qg;      // query tile groups = ceil(T / qpw)
  int xcd_mode;  // 1: workgroups of one kv stream share an XCD (needs B*Hkv % 8 == 0)
  float scale;   // softmax scale
};

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
  constexpr int SUB = 32;
  __shared__ float Ks[SUB][D];
  __shared__ float Vs[SUB][D];
  __shared__ float Ss[SUB][kWave];
  __shared__ int limk[SUB];

  const int lane = threadIdx.x;
  const int qt = a.T - 1 - (int)blockIdx.x;  // heavy query tiles first
  const int bh = blockIdx.y;
  const int b = bh / a.Hq, hq = bh % a.Hq, hkv = hq / a.n_rep;
  const int stream = b * a.Hkv + hkv;
  const int32_t* lim = a.vis_lim + (int64_t)stream * a.S;
  const T* qp = static_cast<const T*>(a.q) + b * a.qs_b + hq * a.qs_h;
  const T* kp = static_cast<const T*>(a.k) + b * a.ks_b + hkv * a.ks_h;
  const T* vp = static_cast<const T*>(a.v) + b * a.vs_b + hkv * a.vs_h;
  T* op = static_cast<T*>(a.o) + b * a.os_b + hq * a.os_h;

  const int m = qt * kTile + lane;
  const bool row_ok = m < a.L;
  const int m_slot = m >> a.c_shift;
  const int m0_slot = (qt * kTile) >> a.c_shift;

  float qv[D], acc[D];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    qv[d] = row_ok ? load_as_f32<T>(qp + (int64_t)m * a.qs_l + d) : 0.f;
    acc[d] = 0.f;
  }
  float m_run = -INFINITY, l_run = 0.f;

  const int last_key = min(qt * kTile + kTile - 1, a.L - 1);
  for (int k0 = 0; k0 <= last_key; k0 += SUB) {
    // does any slot of this sub-tile reach the first query slot of the tile?
    int key = k0 + lane;
    bool reach = lane < SUB && key < a.L && lim[key >> a.c_shift] >= m0_slot;
    if (__ballot(reach) == 0) continue;
    __syncthreads();  // previous sub-tile fully consumed
    for (int idx = lane; idx < SUB * D; idx += kWave) {
      int r = idx / D, d = idx % D;
      int n = k0 + r;
      bool ok = n < a.L;
      Ks[r][d] = ok ? load_as_f32<T>(kp + (int64_t)n * a.ks_l + d) : 0.f;
      Vs[r][d] = ok ? load_as_f32<T>(vp + (int64_t)n * a.vs_l + d) : 0.f;
    }
    if (lane < SUB) limk[lane] = key < a.L ? lim[key >> a.c_shift] : -1;
    __syncthreads();

    float tmax = -INFINITY;
    for (int j = 0; j < SUB; ++j) {
      float dot = 0.f;
#pragma unroll
      for (int d = 0; d < D; ++d) dot = fmaf(qv[d], Ks[j][d], dot);
      int n = k0 + j;
      bool vis = row_ok && n <= m && m_slot <= limk[j];
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
    for (int d = 0; d < D; ++d) store_from_f32<T>(op + (int64_t)m * a.os_l + d, acc[d] * inv);
  }
}

// ---------------------------------------------------------------------------------------------------
// bf16 MFMA kernel.
//
// Workgroup = 4 wavefronts = (hpw q heads of one kv head) x (qpw query tiles of 64 rows); every wavefront
// owns 64 query rows of one q head and all wavefronts share each 64-key K / V tile through LDS.
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

constexpr int kWin = 1024;  // key tiles whose visit list is built at once

template <int D>
struct PrefillSmem {
  uint16_t k[2][kTile * D];
  uint16_t v[2][kTile * D];
  int limk[2][kTile];
  int4 vlist[kWin];  // visited key tiles of the current window: {tile, max vis_lim, min vis_lim, -}
  int vcount;
};

template <int D>
__global__ __launch_bounds__(256) void prefill_mfma_kernel(PrefillArgs a) {
  constexpr int OCT = D / 8;              // 16-byte chunks per row
  constexpr int DMA_PER_WAVE = OCT / 4;   // 1 KiB global->LDS transfers per wavefront and tensor
  constexpr int DSTEPS = D / 16;
  constexpr int DT = D / 32;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  PrefillSmem<D>& sm = *reinterpret_cast<PrefillSmem<D>*>(smem_raw);

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int hl = lane >> 5;

  // ---- which (kv stream, head group, query group) -------------------------------------------------
  int bid = blockIdx.x;
  int ks, hg, rank;
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
  const int qg = a.n_qg - 1 - rank;  // heavy query groups first
  const int b = ks / a.Hkv, hkv = ks % a.Hkv;
  const int hq = hkv * a.n_rep + hg * a.hpw + (wave % a.hpw);
  const int qt_lo = qg * a.qpw;
  const int qt_hi = min(qt_lo + a.qpw - 1, a.T - 1);
  const int my_qt = qt_lo + wave / a.hpw;
  const bool wave_live = my_qt <= qt_hi;
  const int q0 = my_qt * kTile;

  const int2* tl = a.tile_lim + (int64_t)ks * a.T;
  const int32_t* lim = a.vis_lim + (int64_t)ks * a.S;
  const uint16_t* kp = static_cast<const uint16_t*>(a.k) + b * a.ks_b + hkv * a.ks_h;
  const uint16_t* vp = static_cast<const uint16_t*>(a.v) + b * a.vs_b + hkv * a.vs_h;

  const int m0_group = (qt_lo * kTile) >> a.c_shift;
  const int my_m0 = q0 >> a.c_shift;
  const int my_mlast = (min(q0 + kTile - 1, a.L - 1)) >> a.c_shift;

  // ---- Q fragments: B operand, lane (query l32, k-group hl) --------------------------------------
  bf16x8 qreg[2][DSTEPS];
  {
    const uint16_t* qp = static_cast<const uint16_t*>(a.q) + b * a.qs_b + hq * a.qs_h;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      int row = min(q0 + qb * 32 + l32, a.L - 1);
      if (!wave_live) row = 0;
      const uint4* rp = reinterpret_cast<const uint4*>(qp + (int64_t)row * a.qs_l + hl * 8);
#pragma unroll
      for (int s = 0; s < DSTEPS; ++s) qreg[qb][s] = __builtin_bit_cast(bf16x8, rp[s * 2]);
    }
  }

  f32x16 oacc[DT][2];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[dt][qb][i] = 0.f;
  float m_run[2] = {-INFINITY, -INFINITY};
  float l_run[2] = {0.f, 0.f};
  const float c = a.scale * 1.4426950408889634f;

  // global -> LDS, one 64-key tile of K and of V; rows beyond L repeat row L-1 (their scores are masked,
  // so their probabilities are exactly 0 and a finite V row contributes nothing)
  auto issue_tile = [&](int kt, int buf, bool need_lim) {
#pragma unroll
    for (int j = 0; j < DMA_PER_WAVE; ++j) {
      const int inst = wave * DMA_PER_WAVE + j;  // uniform
      const int q = inst * kWave + lane;         // chunk slot in the LDS tile
      const int row = q / OCT, pos = q % OCT;
      const int n = min(kt * kTile + row, a.L - 1);
      const int kchunk = pos ^ (row % OCT);
      const int vchunk = pos ^ ((row & 3) << 1);
      __builtin_amdgcn_global_load_lds(kp + (int64_t)n * a.ks_l + kchunk * 8,
                                       (uint32_t __attribute__((address_space(3)))*)(&sm.k[buf][inst * kWave * 8]), 16, 0, 0);
      __builtin_amdgcn_global_load_lds(vp + (int64_t)n * a.vs_l + vchunk * 8,
                                       (uint32_t __attribute__((address_space(3)))*)(&sm.v[buf][inst * kWave * 8]), 16, 0, 0);
    }
    if (need_lim && tid < kTile) {
      int n = kt * kTile + tid;
      sm.limk[buf][tid] = n < a.L ? lim[n >> a.c_shift] : -1;
    }
  };

  auto compute_tile = [&](int kt, int cur, bool full) {
    const uint16_t* Kt = sm.k[cur];
    const uint16_t* Vt = sm.v[cur];
    // ---- S^T = K Q^T ---------------------------------------------------------------------------
    f32x16 sacc[2][2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const int row = kb * 32 + l32;
#pragma unroll
      for (int s = 0; s < DSTEPS; ++s) {
        const int chunk = (s * 2 + hl) ^ (row % OCT);
        bf16x8 ka = *reinterpret_cast<const bf16x8*>(Kt + row * D + chunk * 8);
        if (s == 0) {
          const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          sacc[kb][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qreg[0][s], z, 0, 0, 0);
          sacc[kb][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qreg[1][s], z, 0, 0, 0);
        } else {
          sacc[kb][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qreg[0][s], sacc[kb][0], 0, 0, 0);
          sacc[kb][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qreg[1][s], sacc[kb][1], 0, 0, 0);
        }
      }
    }
    // ---- mask (diagonal tile, or a tile whose slots are not uniformly visible) -----------------
    if (!full) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          int kk = kb * 32 + g4 * 8 + hl * 4;  // key offset in tile of accumulator 4*g4
          int4 lm = *reinterpret_cast<const int4*>(&sm.limk[cur][kk]);
          const int lv[4] = {lm.x, lm.y, lm.z, lm.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            int key = kt * kTile + kk + e;
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
              int qtok = q0 + qb * 32 + l32;
              bool vis = key <= qtok && (qtok >> a.c_shift) <= lv[e];
              if (!vis) sacc[kb][qb][g4 * 4 + e] = -INFINITY;
            }
          }
        }
      }
    }
    // ---- online softmax, one query per lane and q block ----------------------------------------
    bf16x8 pb[2][4];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      float mx = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, sacc[kb][qb][i]);
      mx = fmaxf(mx, __shfl_xor(mx, 32)) * c;
      if (__ballot(mx > m_run[qb] + kRescaleSlack)) {
        float m_new = fmaxf(m_run[qb], mx);
        float alpha = m_run[qb] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run[qb] - m_new);
        l_run[qb] *= alpha;
        m_run[qb] = m_new;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) oacc[dt][qb][i] *= alpha;
      }
      const float m_use = m_run[qb] == -INFINITY ? 0.f : m_run[qb];
      float rs = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float p = __builtin_amdgcn_exp2f(fmaf(sacc[kb][qb][i], c, -m_use));
          rs += p;
          pb[qb][kb * 2 + (i >> 3)][i & 7] = (__bf16)p;
        }
      }
      l_run[qb] += rs;
    }
    // ---- O^T += V^T P^T ------------------------------------------------------------------------
    // ds_read_b64_tr_b16: within 16 lanes, lane r reads 4 dims of key (K0 + r / 4) starting at dim
    // D0 + 4 * (r % 4) and receives keys K0 .. K0 + 3 of dim D0 + r.
    const int r16 = lane & 15;
    const int dsel = (lane >> 4) & 1;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const int chunk0 = dt * 4 + dsel * 2 + ((r16 & 3) >> 1);
      const int half = r16 & 1;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        bf16x4 lo, hi;
        {
          const int row = t * 16 + hl * 4 + (r16 >> 2);
          const uint16_t* pa = Vt + row * D + ((chunk0 ^ ((row & 3) << 1)) * 8) + half * 4;
          lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4 __attribute__((address_space(3)))*)pa);
        }
        {
          const int row = t * 16 + 8 + hl * 4 + (r16 >> 2);
          const uint16_t* pa = Vt + row * D + ((chunk0 ^ ((row & 3) << 1)) * 8) + half * 4;
          hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4 __attribute__((address_space(3)))*)pa);
        }
        bf16x8 va = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        oacc[dt][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb[0][t], oacc[dt][0], 0, 0, 0);
        oacc[dt][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb[1][t], oacc[dt][1], 0, 0, 0);
      }
    }
  };

  const int mlast_group = (min(qt_hi * kTile + kTile - 1, a.L - 1)) >> a.c_shift;
  int cur = 0;
  for (int w0 = 0; w0 <= qt_hi; w0 += kWin) {
    // ---- visit list of this window: wavefront 0 compacts the tiles some query tile of the group sees ----
    if (wave == 0) {
      int2 vals[kWin / kWave];
#pragma unroll
      for (int j = 0; j < kWin / kWave; ++j) {
        int t = w0 + j * kWave + lane;
        vals[j] = t <= qt_hi ? tl[t] : make_int2(-1, -1);
      }
      int count = 0;
#pragma unroll
      for (int j = 0; j < kWin / kWave; ++j) {
        int t = w0 + j * kWave + lane;
        bool v = t <= qt_hi && vals[j].x >= m0_group;
        uint64_t bits = __ballot(v);
        if (v) sm.vlist[count + __builtin_popcountll(bits & ((uint64_t(1) << lane) - 1))] = make_int4(t, vals[j].x, vals[j].y, 0);
        count += __builtin_popcountll(bits);
      }
      if (lane == 0) sm.vcount = count;
    }
    __syncthreads();
    const int n_vis = sm.vcount;
    if (n_vis > 0) {
      issue_tile(sm.vlist[0].x, cur, true);
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
    }
    for (int idx = 0; idx < n_vis; ++idx) {
      const int4 ent = sm.vlist[idx];
      const int kt = ent.x;
      if (idx + 1 < n_vis) {
        const int4 en = sm.vlist[idx + 1];
        // the element mask is only evaluated on diagonal tiles and on tiles with mixed visibility
        issue_tile(en.x, cur ^ 1, en.x >= qt_lo || en.z < mlast_group);
      }
      const bool visit = wave_live && kt <= my_qt && ent.y >= my_m0;
      if (visit) {
        const bool full = kt < my_qt && ent.z >= my_mlast;
        compute_tile(kt, cur, full);
      }
      __builtin_amdgcn_s_waitcnt(0);  // the next tile has landed in LDS
      __syncthreads();                // ... for every wavefront, and this tile is no longer read
      cur ^= 1;
    }
  }

  // ---- epilogue -----------------------------------------------------------------------------------
  if (wave_live) {
    uint16_t* op = static_cast<uint16_t*>(a.o) + b * a.os_b + hq * a.os_h;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      float l = l_run[qb] + __shfl_xor(l_run[qb], 32);
      float inv = 1.f / l;
      int qtok = q0 + qb * 32 + l32;
      if (qtok < a.L) {
        uint16_t* rp = op + (int64_t)qtok * a.os_l;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4) {
            int d = dt * 32 + g4 * 8 + hl * 4;
            uint32_t lo = uint32_t(f32_to_bf16_bits(oacc[dt][qb][g4 * 4 + 0] * inv)) |
                          (uint32_t(f32_to_bf16_bits(oacc[dt][qb][g4 * 4 + 1] * inv)) << 16);
            uint32_t hi = uint32_t(f32_to_bf16_bits(oacc[dt][qb][g4 * 4 + 2] * inv)) |
                          (uint32_t(f32_to_bf16_bits(oacc[dt][qb][g4 * 4 + 3] * inv)) << 16);
            *reinterpret_cast<uint2*>(rp + d) = make_uint2(lo, hi);
          }
        }
      }
    }
  }
}

template <int D>
static int launch_prefill_mfma(const PrefillArgs& a, int64_t n_wg, hipStream_t st) {
  static bool configured = false;  // per process and head size; the attribute is a property of the kernel
  const size_t smem = sizeof(PrefillSmem<D>);
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_mfma_kernel<D>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return fail(NATS_ERR_LAUNCH, "hipFuncSetAttribute(%zu bytes of LDS): %s", smem, hipGetErrorString(e));
    configured = true;
  }
  hipLaunchKernelGGL((prefill_mfma_kernel<D>), dim3((unsigned)n_wg), dim3(256), smem, st, a);
  NATS_CHECK_LAUNCH("prefill_mfma_kernel");
  return NATS_OK;
}

}  // namespace nats

using namespace nats;

extern "C" size_t nats_prefill_workspace_bytes(int64_t B, int64_t H_q, int64_t H_kv, int64_t L, int64_t D, int64_t C) {
  (void)H_q;
  (void)D;
  if (B <= 0 || H_kv <= 0 || L <= 0 || C <= 0) return 0;
  int64_t S = (L + C - 1) / C;
  int64_t T = (L + kTile - 1) / kTile;
  size_t lim_bytes = ((size_t)(B * H_kv * S) * sizeof(int32_t) + 255) & ~size_t(255);
  size_t tl_bytes = (size_t)(B * H_kv * T) * sizeof(int2);
  return lim_bytes + tl_bytes;
}

extern "C" int nats_prefill_fwd(const void* q, const void* k, const void* v, const uint8_t* roles, void* o, int64_t B,
                                int64_t H_q, int64_t H_kv, int64_t L, int64_t D, int64_t C, int64_t W,
                                const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                const int64_t* o_strides, float sm_scale, int dtype, void* workspace,
                                size_t workspace_bytes, void* stream) {
  NATS_REQUIRE(q && k && v && roles && o && workspace, NATS_ERR_NULL_POINTER, "nats_prefill_fwd: NULL pointer argument");
  NATS_REQUIRE(q_strides && k_strides && v_strides && o_strides, NATS_ERR_NULL_POINTER,
               "nats_prefill_fwd: NULL stride array");
  NATS_REQUIRE(B > 0 && H_q > 0 && H_kv > 0 && L > 0, NATS_ERR_BAD_SHAPE, "nats_prefill_fwd: B=%lld H_q=%lld H_kv=%lld L=%lld",
               (long long)B, (long long)H_q, (long long)H_kv, (long long)L);
  NATS_REQUIRE(H_q % H_kv == 0, NATS_ERR_BAD_SHAPE, "nats_prefill_fwd: H_q=%lld is not a multiple of H_kv=%lld",
               (long long)H_q, (long long)H_kv);
  NATS_REQUIRE(D == 64 || D == 128, NATS_ERR_UNSUPPORTED, "nats_prefill_fwd: head_dim %lld (supported: 64, 128)",
               (long long)D);
  NATS_REQUIRE(is_pow2(C), NATS_ERR_UNSUPPORTED, "nats_prefill_fwd: chunk size %lld is not a power of two", (long long)C);
  NATS_REQUIRE(W >= 0 && W % C == 0, NATS_ERR_BAD_SHAPE, "nats_prefill_fwd: window %lld is not a multiple of chunk size %lld",
               (long long)W, (long long)C);
  NATS_REQUIRE(dtype == NATS_DTYPE_BF16 || dtype == NATS_DTYPE_F32, NATS_ERR_BAD_DTYPE, "nats_prefill_fwd: dtype %d", dtype);
  NATS_REQUIRE(L < (int64_t(1) << 30), NATS_ERR_BAD_SHAPE, "nats_prefill_fwd: L=%lld too long", (long long)L);
  size_t need = nats_prefill_workspace_bytes(B, H_q, H_kv, L, D, C);
  NATS_REQUIRE(workspace_bytes >= need, NATS_ERR_WORKSPACE, "nats_prefill_fwd: workspace %zu bytes < %zu", workspace_bytes,
               need);
  if (dtype == NATS_DTYPE_BF16) {
    // 16-byte vector loads of rows
    NATS_REQUIRE(q_strides[2] % 8 == 0 && k_strides[2] % 8 == 0 && v_strides[2] % 8 == 0 && o_strides[2] % 4 == 0 &&
                     q_strides[1] % 8 == 0 && k_strides[1] % 8 == 0 && v_strides[1] % 8 == 0 && o_strides[1] % 4 == 0 &&
                     q_strides[0] % 8 == 0 && k_strides[0] % 8 == 0 && v_strides[0] % 8 == 0 && o_strides[0] % 4 == 0,
                 NATS_ERR_BAD_SHAPE, "nats_prefill_fwd: bf16 strides must keep rows 16-byte aligned");
    NATS_REQUIRE((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v)) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(o) % 8 == 0,
                 NATS_ERR_BAD_SHAPE, "nats_prefill_fwd: bf16 tensors must be 16-byte aligned");
  }

  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t S = (L + C - 1) / C;
  const int64_t T = (L + kTile - 1) / kTile;
  int32_t* vis_lim = static_cast<int32_t*>(workspace);
  size_t lim_bytes = ((size_t)(B * H_kv * S) * sizeof(int32_t) + 255) & ~size_t(255);
  int2* tile_lim = reinterpret_cast<int2*>(static_cast<char*>(workspace) + lim_bytes);
  if (int rc = launch_role_scan(roles, B * H_kv, S, W, C, nullptr, vis_lim, st)) return rc;
  if (int rc = launch_tile_lim(vis_lim, B * H_kv, S, T, C, tile_lim, st)) return rc;

  PrefillArgs a;
  a.q = q; a.k = k; a.v = v; a.o = o;
  a.vis_lim = vis_lim; a.tile_lim = tile_lim;
  a.qs_b = q_strides[0]; a.qs_h = q_strides[1]; a.qs_l = q_strides[2];
  a.ks_b = k_strides[0]; a.ks_h = k_strides[1]; a.ks_l = k_strides[2];
  a.vs_b = v_strides[0]; a.vs_h = v_strides[1]; a.vs_l = v_strides[2];
  a.os_b = o_strides[0]; a.os_h = o_strides[1]; a.os_l = o_strides[2];
  a.B = (int)B; a.Hq = (int)H_q; a.Hkv = (int)H_kv; a.n_rep = (int)(H_q / H_kv);
  a.L = (int)L; a.S = (int)S; a.T = (int)T;
  a.c_shift = ilog2(C);
  a.scale = sm_scale;
  a.hpw = 1; a.qpw = 1; a.n_hg = 1; a.n_qg = (int)T; a.xcd_mode = 0;

  if (dtype == NATS_DTYPE_F32) {
    NATS_REQUIRE(B * H_q <= 65535, NATS_ERR_BAD_SHAPE, "nats_prefill_fwd: B*H_q too large for the fp32 kernel");
    dim3 grid((unsigned)T, (unsigned)(B * H_q));
    if (D == 64) {
      hipLaunchKernelGGL((prefill_simple_kernel<float, 64>), grid, dim3(64), 0, st, a);
    } else {
      hipLaunchKernelGGL((prefill_simple_kernel<float, 128>), grid, dim3(64), 0, st, a);
    }
    NATS_CHECK_LAUNCH("prefill_simple_kernel");
    return NATS_OK;
  }

  // bf16: pack the q heads of one kv head into one workgroup (up to 4), fill the rest with query tiles
  int n_rep = a.n_rep;
  int hpw = n_rep >= 4 ? 4 : n_rep;
  NATS_REQUIRE(n_rep % hpw == 0 && (4 % hpw) == 0, NATS_ERR_UNSUPPORTED,
               "nats_prefill_fwd: GQA group size %d (supported: 1, 2, 4 and multiples of 4)", n_rep);
  a.hpw = hpw;
  a.qpw = 4 / hpw;
  a.n_hg = n_rep / hpw;
  a.n_qg = (int)((T + a.qpw - 1) / a.qpw);
  a.xcd_mode = ((B * H_kv) % 8 == 0) ? 1 : 0;
  int64_t n_wg = B * H_kv * a.n_hg * a.n_qg;
  NATS_REQUIRE(n_wg < (int64_t(1) << 31), NATS_ERR_BAD_SHAPE, "nats_prefill_fwd: grid too large");
  return D == 64 ? launch_prefill_mfma<64>(a, n_wg, st) : launch_prefill_mfma<128>(a, n_wg, st);
}
