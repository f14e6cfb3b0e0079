// One-token decode attention over the evicted, ragged KV cache (HBM bound).
//
// Semantics: o[b, hq] = softmax over the rows i < n_rows with valid[b, hkv, i] != 0 of q . K[i] * scale, times V.
// (components/cache/nats_chunk_layer_cache.py:622-632 + SDPA; models/transformer/hf/llama.py:274-295.)
// Rows whose valid byte is 0 are never loaded, so whatever sits between a head's own end and the
// batch-wide n_ctx_data costs no bandwidth.
//
// Split-K: grid = (splits of the row range) x (b, kv head) x (groups of q heads).  Inside a workgroup the
// four wavefronts take interleaved 64-row tiles, keep (m, l, acc) per q head and are merged through LDS;
// one partial per workgroup goes to the workspace and a second small kernel merges the splits.
#include "nats_common.h"

namespace nats {

struct DecodeArgs {
  const void* q;
  const void* k;
  const void* v;
  const uint8_t* valid;
  void* o;
  float* ws_acc;  // [B*Hq, nsplit, D]
  float* ws_ml;   // [B*Hq, nsplit, 2]
  int64_t ks_b, ks_h, ks_r;
  int64_t vs_b, vs_h;
  int B, Hq, Hkv, n_rep;
  int n_rows, rows_per_split, nsplit;
  float scale;
};

__device__ __forceinline__ float exp2_guard(float x) { return __builtin_amdgcn_exp2f(x); }

// ---------------------------------------------------------------------------------------------------
// bf16: S^T = K Q^T on v_mfma_f32_16x16x32_bf16 (A = 16 key rows straight from global memory, B = the q
// heads of the group padded to 16 columns), softmax per q head, probabilities broadcast through
// wave-private LDS, PV on the vector ALU with fully coalesced 16-byte V loads.
// ---------------------------------------------------------------------------------------------------
template <int D, int NREP>
__global__ __launch_bounds__(256) void decode_split_mfma_kernel(DecodeArgs a) {
  constexpr int STEPS = D / 32;
  constexpr int LPR = D / 8;    // lanes per V row
  constexpr int RPI = 64 / LPR; // V rows per load instruction
  constexpr int NVL = 64 / RPI; // V loads per tile

  __shared__ float p_lds[4][64][NREP];
  __shared__ float al_lds[4][NREP];
  __shared__ float wacc[4][NREP][D];
  __shared__ float wm[4][NREP];
  __shared__ float wl[4][NREP];

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int l16 = lane & 15;
  const int lg = lane >> 4;

  const int split = blockIdx.x;
  const int ks = blockIdx.y;  // b * Hkv + hkv
  const int grp = blockIdx.z;
  const int b = ks / a.Hkv, hkv = ks % a.Hkv;
  const int hq0 = hkv * a.n_rep + grp * NREP;

  const uint16_t* kp = static_cast<const uint16_t*>(a.k) + b * a.ks_b + hkv * a.ks_h;
  const uint16_t* vp = static_cast<const uint16_t*>(a.v) + b * a.ks_b + hkv * a.ks_h;
  const uint8_t* valp = a.valid + b * a.vs_b + hkv * a.vs_h;

  // Q as the B operand: column = q head of the group (zero beyond NREP), k = 8 dims per lane group
  bf16x8 qreg[STEPS];
  {
    const uint16_t* qp = static_cast<const uint16_t*>(a.q) + ((int64_t)b * a.Hq + hq0 + (l16 < NREP ? l16 : 0)) * D;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      uint4 raw = *reinterpret_cast<const uint4*>(qp + s * 32 + lg * 8);
      if (l16 >= NREP) raw = make_uint4(0, 0, 0, 0);
      qreg[s] = __builtin_bit_cast(bf16x8, raw);
    }
  }

  float acc[NREP][8];
#pragma unroll
  for (int h = 0; h < NREP; ++h)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[h][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;  // of q head l16 (meaningful for l16 < NREP)
  const float c = a.scale * 1.4426950408889634f;

  const int r_begin = split * a.rows_per_split;
  const int r_end = min(r_begin + a.rows_per_split, a.n_rows);

  for (int row0 = r_begin + wave * 64; row0 < r_end; row0 += 256) {
    bool vb = (row0 + lane < r_end) && valp[row0 + lane] != 0;
    const uint64_t vmask = __ballot(vb);
    if (vmask == 0) continue;

    uint4 kreg[4][STEPS];
    uint4 vreg[NVL];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      int kl = g * 16 + l16;
      bool ok = (vmask >> kl) & 1;
      const uint16_t* rp = kp + (int64_t)(row0 + kl) * a.ks_r + lg * 8;
#pragma unroll
      for (int s = 0; s < STEPS; ++s) {
        kreg[g][s] = ok ? *reinterpret_cast<const uint4*>(rp + s * 32) : make_uint4(0, 0, 0, 0);
      }
    }
#pragma unroll
    for (int j = 0; j < NVL; ++j) {
      int kl = j * RPI + lane / LPR;
      bool ok = (vmask >> kl) & 1;
      vreg[j] = ok ? *reinterpret_cast<const uint4*>(vp + (int64_t)(row0 + kl) * a.ks_r + (lane % LPR) * 8)
                   : make_uint4(0, 0, 0, 0);
    }

    // scores: sc[g][i] belongs to key g*16 + lg*4 + i and q head l16
    float sc[4][4];
    float mx = -INFINITY;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < STEPS; ++s) {
        s4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kreg[g][s]), qreg[s], s4, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int kl = g * 16 + lg * 4 + i;
        float sv = ((vmask >> kl) & 1) ? s4[i] : -INFINITY;
        sc[g][i] = sv;
        mx = fmaxf(mx, sv);
      }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    float m_new = fmaxf(m_run, mx * c);  // vmask != 0, so mx is finite
    float alpha = exp2_guard(m_run - m_new);
    float rs = 0.f;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float p = exp2_guard(fmaf(sc[g][i], c, -m_new));
        rs += p;
        if (l16 < NREP) p_lds[wave][g * 16 + lg * 4 + i][l16] = p;
      }
    }
    l_run = l_run * alpha + rs;
    m_run = m_new;
    if (lane < NREP) al_lds[wave][lane] = alpha;
    wave_lds_sync();

    float al[NREP];
#pragma unroll
    for (int h = 0; h < NREP; ++h) al[h] = al_lds[wave][h];
#pragma unroll
    for (int h = 0; h < NREP; ++h)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[h][e] *= al[h];
#pragma unroll
    for (int j = 0; j < NVL; ++j) {
      int kl = j * RPI + lane / LPR;
      float ph[NREP];
#pragma unroll
      for (int h = 0; h < NREP; ++h) ph[h] = p_lds[wave][kl][h];
      const uint32_t w[4] = {vreg[j].x, vreg[j].y, vreg[j].z, vreg[j].w};
#pragma unroll
      for (int e2 = 0; e2 < 4; ++e2) {
        float v0 = __uint_as_float(w[e2] << 16);
        float v1 = __uint_as_float(w[e2] & 0xffff0000u);
#pragma unroll
        for (int h = 0; h < NREP; ++h) {
          acc[h][2 * e2] = fmaf(ph[h], v0, acc[h][2 * e2]);
          acc[h][2 * e2 + 1] = fmaf(ph[h], v1, acc[h][2 * e2 + 1]);
        }
      }
    }
    wave_lds_sync();
  }

  // ---- merge the lane groups of a wavefront, then the wavefronts of the workgroup --------------------
#pragma unroll
  for (int h = 0; h < NREP; ++h) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float x = acc[h][e];
      if (LPR < 16) x += __shfl_xor(x, 8);
      x += __shfl_xor(x, 16);
      x += __shfl_xor(x, 32);
      acc[h][e] = x;
    }
  }
  l_run += __shfl_xor(l_run, 16);
  l_run += __shfl_xor(l_run, 32);
  if (lane < LPR) {
#pragma unroll
    for (int h = 0; h < NREP; ++h)
#pragma unroll
      for (int e = 0; e < 8; ++e) wacc[wave][h][lane * 8 + e] = acc[h][e];
  }
  if (lane < NREP) {
    wm[wave][lane] = m_run;
    wl[wave][lane] = l_run;
  }
  __syncthreads();
  for (int idx = tid; idx < NREP * D; idx += 256) {
    int h = idx / D, d = idx % D;
    float M = fmaxf(fmaxf(wm[0][h], wm[1][h]), fmaxf(wm[2][h], wm[3][h]));
    float sum = 0.f, lsum = 0.f;
    if (M != -INFINITY) {
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        float f = exp2_guard(wm[w][h] - M);
        sum += wacc[w][h][d] * f;
        lsum += wl[w][h] * f;
      }
    }
    int64_t head = (int64_t)b * a.Hq + hq0 + h;
    a.ws_acc[(head * a.nsplit + split) * D + d] = sum;
    if (d == 0) {
      a.ws_ml[(head * a.nsplit + split) * 2 + 0] = M;
      a.ws_ml[(head * a.nsplit + split) * 2 + 1] = lsum;
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// fp32: one q head per workgroup, one key row per wavefront step; the parity path for fp32 caches.
// ---------------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void decode_split_f32_kernel(DecodeArgs a) {
  constexpr int PER = D / 64;
  __shared__ float wacc[4][D];
  __shared__ float wm[4];
  __shared__ float wl[4];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int split = blockIdx.x;
  const int head = blockIdx.y;  // b * Hq + hq
  const int b = head / a.Hq, hq = head % a.Hq, hkv = hq / a.n_rep;
  const float* kp = static_cast<const float*>(a.k) + b * a.ks_b + hkv * a.ks_h;
  const float* vp = static_cast<const float*>(a.v) + b * a.ks_b + hkv * a.ks_h;
  const uint8_t* valp = a.valid + b * a.vs_b + hkv * a.vs_h;
  const float* qp = static_cast<const float*>(a.q) + (int64_t)head * D;
  float qv[PER], acc[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    qv[e] = qp[lane * PER + e];
    acc[e] = 0.f;
  }
  float m_run = -INFINITY, l_run = 0.f;
  const int r_begin = split * a.rows_per_split;
  const int r_end = min(r_begin + a.rows_per_split, a.n_rows);
  for (int r = r_begin + wave; r < r_end; r += 4) {
    if (valp[r] == 0) continue;
    const float* kr = kp + (int64_t)r * a.ks_r;
    const float* vr = vp + (int64_t)r * a.ks_r;
    float dot = 0.f;
#pragma unroll
    for (int e = 0; e < PER; ++e) dot = fmaf(qv[e], kr[lane * PER + e], dot);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off);
    float s = dot * a.scale;
    float m_new = fmaxf(m_run, s);
    float alpha = expf(m_run - m_new);
    float p = expf(s - m_new);
    l_run = l_run * alpha + p;
#pragma unroll
    for (int e = 0; e < PER; ++e) acc[e] = fmaf(p, vr[lane * PER + e], acc[e] * alpha);
    m_run = m_new;
  }
#pragma unroll
  for (int e = 0; e < PER; ++e) wacc[wave][lane * PER + e] = acc[e];
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
  *nsplit = (int)((n_rows + r - 1) / r);
}

template <int D, int NREP>
static void launch_mfma(const DecodeArgs& a, int groups, hipStream_t st) {
  dim3 grid((unsigned)a.nsplit, (unsigned)(a.B * a.Hkv), (unsigned)groups);
  hipLaunchKernelGGL((decode_split_mfma_kernel<D, NREP>), grid, dim3(256), 0, st, a);
}

}  // namespace nats

using namespace nats;

extern "C" size_t nats_decode_workspace_bytes(int64_t B, int64_t H_q, int64_t H_kv, int64_t D, int64_t n_rows) {
  if (B <= 0 || H_q <= 0 || H_kv <= 0 || D <= 0 || n_rows <= 0) return 0;
  int rps, ns;
  decode_split_geometry(B, H_kv, n_rows, &rps, &ns);
  return (size_t)B * H_q * ns * (D + 2) * sizeof(float);
}

extern "C" int nats_decode_fwd(const void* q, const void* cache_k, const void* cache_v, const uint8_t* valid, void* o,
                               int64_t B, int64_t H_q, int64_t H_kv, int64_t D, int64_t n_rows, const int64_t* kv_strides,
                               const int64_t* valid_strides, float sm_scale, int dtype, void* workspace,
                               size_t workspace_bytes, void* stream) {
  NATS_REQUIRE(q && cache_k && cache_v && valid && o && workspace, NATS_ERR_NULL_POINTER,
               "nats_decode_fwd: NULL pointer argument");
  NATS_REQUIRE(kv_strides && valid_strides, NATS_ERR_NULL_POINTER, "nats_decode_fwd: NULL stride array");
  NATS_REQUIRE(B > 0 && H_q > 0 && H_kv > 0 && n_rows > 0, NATS_ERR_BAD_SHAPE,
               "nats_decode_fwd: B=%lld H_q=%lld H_kv=%lld n_rows=%lld", (long long)B, (long long)H_q, (long long)H_kv,
               (long long)n_rows);
  NATS_REQUIRE(H_q % H_kv == 0, NATS_ERR_BAD_SHAPE, "nats_decode_fwd: H_q=%lld is not a multiple of H_kv=%lld",
               (long long)H_q, (long long)H_kv);
  NATS_REQUIRE(D == 64 || D == 128, NATS_ERR_UNSUPPORTED, "nats_decode_fwd: head_dim %lld (supported: 64, 128)",
               (long long)D);
  NATS_REQUIRE(dtype == NATS_DTYPE_BF16 || dtype == NATS_DTYPE_F32, NATS_ERR_BAD_DTYPE, "nats_decode_fwd: dtype %d", dtype);
  NATS_REQUIRE(n_rows < (int64_t(1) << 30) && B * H_q <= (int64_t(1) << 30), NATS_ERR_BAD_SHAPE,
               "nats_decode_fwd: problem too large");
  NATS_REQUIRE(B * H_kv <= 65535 && B * H_q <= 65535 * 16, NATS_ERR_BAD_SHAPE, "nats_decode_fwd: too many (b, head) streams");
  size_t need = nats_decode_workspace_bytes(B, H_q, H_kv, D, n_rows);
  NATS_REQUIRE(workspace_bytes >= need, NATS_ERR_WORKSPACE, "nats_decode_fwd: workspace %zu bytes < %zu", workspace_bytes,
               need);
  if (dtype == NATS_DTYPE_BF16) {
    NATS_REQUIRE(kv_strides[0] % 8 == 0 && kv_strides[1] % 8 == 0 && kv_strides[2] % 8 == 0, NATS_ERR_BAD_SHAPE,
                 "nats_decode_fwd: bf16 cache strides must keep rows 16-byte aligned");
    NATS_REQUIRE((reinterpret_cast<uintptr_t>(cache_k) | reinterpret_cast<uintptr_t>(cache_v) |
                  reinterpret_cast<uintptr_t>(q)) % 16 == 0,
                 NATS_ERR_BAD_SHAPE, "nats_decode_fwd: bf16 tensors must be 16-byte aligned");
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  DecodeArgs a;
  a.q = q; a.k = cache_k; a.v = cache_v; a.valid = valid; a.o = o;
  a.ks_b = kv_strides[0]; a.ks_h = kv_strides[1]; a.ks_r = kv_strides[2];
  a.vs_b = valid_strides[0]; a.vs_h = valid_strides[1];
  a.B = (int)B; a.Hq = (int)H_q; a.Hkv = (int)H_kv; a.n_rep = (int)(H_q / H_kv);
  a.n_rows = (int)n_rows;
  decode_split_geometry(B, H_kv, n_rows, &a.rows_per_split, &a.nsplit);
  a.scale = sm_scale;
  a.ws_acc = static_cast<float*>(workspace);
  a.ws_ml = a.ws_acc + (size_t)B * H_q * a.nsplit * D;

  if (dtype == NATS_DTYPE_F32) {
    dim3 grid((unsigned)a.nsplit, (unsigned)(B * H_q));
    if (D == 64) {
      hipLaunchKernelGGL((decode_split_f32_kernel<64>), grid, dim3(256), 0, st, a);
    } else {
      hipLaunchKernelGGL((decode_split_f32_kernel<128>), grid, dim3(256), 0, st, a);
    }
    NATS_CHECK_LAUNCH("decode_split_f32_kernel");
    hipLaunchKernelGGL((decode_merge_kernel<false>), dim3((unsigned)(B * H_q)), dim3((unsigned)D), 0, st, a.ws_acc, a.ws_ml,
                       o, a.nsplit, (int)D);
    NATS_CHECK_LAUNCH("decode_merge_kernel");
    return NATS_OK;
  }

  int n_rep = a.n_rep;
  int nrep_k = (n_rep % 8 == 0) ? 8 : (n_rep % 4 == 0) ? 4 : (n_rep % 2 == 0) ? 2 : 1;
  int groups = n_rep / nrep_k;
  if (D == 128) {
    switch (nrep_k) {
      case 8: launch_mfma<128, 8>(a, groups, st); break;
      case 4: launch_mfma<128, 4>(a, groups, st); break;
      case 2: launch_mfma<128, 2>(a, groups, st); break;
      default: launch_mfma<128, 1>(a, groups, st); break;
    }
  } else {
    switch (nrep_k) {
      case 8: launch_mfma<64, 8>(a, groups, st); break;
      case 4: launch_mfma<64, 4>(a, groups, st); break;
      case 2: launch_mfma<64, 2>(a, groups, st); break;
      default: launch_mfma<64, 1>(a, groups, st); break;
    }
  }
  NATS_CHECK_LAUNCH("decode_split_mfma_kernel");
  hipLaunchKernelGGL((decode_merge_kernel<true>), dim3((unsigned)(B * H_q)), dim3((unsigned)D), 0, st, a.ws_acc, a.ws_ml, o,
                     a.nsplit, (int)D);
  NATS_CHECK_LAUNCH("decode_merge_kernel");
  return NATS_OK;
}
