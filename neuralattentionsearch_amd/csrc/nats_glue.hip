// Small fused kernels around the attention of a decode step, so that a decoder layer of the HF-shaped caller
// costs a dozen launches instead of fifty: residual add + RMSNorm (+ the running chunk statistic of the role
// step), rotary embedding + cache append, SiLU gate.
//
// Each follows the rounding points of the torch ops the reference runs, so that in bf16 the results equal those
// ops element for element wherever the arithmetic is elementwise:
//   * RMSNorm: models/transformer/components.py:14-26 (the HF LlamaRMSNorm form: normalise in fp32, cast to the
//     input dtype, then multiply by the weight in that dtype); the mean of squares is an fp32 reduction whose
//     order differs from the library's.
//   * running chunk statistic: NAtSCache.merge_new_x_values_in_chunk (components/cache/dyn_cache.py:98-115),
//     called for an open chunk by update_nats_cached_x_in_chunk (:117-124) from hf/llama_nats_chunk.py:198.
//   * rotary embedding: transformers' apply_rotary_pos_emb as imported by hf/llama_nats_chunk.py:7 and called at
//     :227 (q * cos + rotate_half(q) * sin, every product and the sum rounded to the dtype), followed by the
//     row write of NAtSChunkLayerCache.update (components/cache/nats_chunk_layer_cache.py:243-256).
//   * SiLU gate: act_fn(gate_proj(x)) * up_proj(x) of the HF Llama MLP the reference keeps unchanged.
//   * matrix-vector products: the nn.Linear projections of a one-token step (hf/llama_nats_chunk.py:185-187 q / k / v,
//     :290 o_proj, and the gate / up / down projections of the HF Llama MLP), fp32 accumulation over k, one
//     rounding to the dtype at the end, as the library GEMM does; the order of the fp32 sum differs from the library's.
#include <type_traits>

#include "nats_common.h"

namespace nats {

template <bool kBf16>
__device__ __forceinline__ float g_load(const void* p, int64_t i) {
  if (kBf16) return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
  return static_cast<const float*>(p)[i];
}
template <bool kBf16>
__device__ __forceinline__ float g_round(float v) {
  return kBf16 ? bf16_bits_to_f32(f32_to_bf16_bits(v)) : v;
}
template <bool kBf16>
__device__ __forceinline__ void g_store(void* p, int64_t i, float v) {
  if (kBf16) {
    static_cast<uint16_t*>(p)[i] = f32_to_bf16_bits(v);
  } else {
    static_cast<float*>(p)[i] = v;
  }
}

struct AddNormArgs {
  void* x;            // [rows, dim] in / out (x += delta)
  const void* delta;  // [rows, dim] or null
  const void* weight; // [dim]
  void* out;          // [rows, dim]
  void* carry;        // [rows, dim] or null
  int dim;
  int carry_mode;     // 0 none, 1 mean (first token of the chunk), 2 mean (later token), 3 max (first), 4 max (later)
  float eps, chunk;
};

// One workgroup of 256 threads per row; the row is kept in registers between the two passes.  VEC consecutive
// columns per thread and step: 8 (16-byte loads of bf16, two 16-byte loads of fp32) when dim % 8 == 0, else 1.
constexpr int kNormThreads = 256;
constexpr int kNormMaxDim = 8192;

template <bool kBf16, int VEC>
__device__ __forceinline__ void load_vec(const void* p, int64_t i, float (&v)[VEC]) {
  if (VEC == 8 && kBf16) {
    const uint4 u = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(p) + i);
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[2 * e] = __uint_as_float(w[e] << 16);
      v[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
    }
  } else if (VEC == 8) {
    const float4 a = *reinterpret_cast<const float4*>(static_cast<const float*>(p) + i);
    const float4 b = *reinterpret_cast<const float4*>(static_cast<const float*>(p) + i + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  } else {
#pragma unroll
    for (int e = 0; e < VEC; ++e) v[e] = g_load<kBf16>(p, i + e);
  }
}
template <bool kBf16, int VEC>
__device__ __forceinline__ void store_vec(void* p, int64_t i, const float (&v)[VEC]) {
  if (VEC == 8 && kBf16) {
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = uint32_t(f32_to_bf16_bits(v[2 * e])) | (uint32_t(f32_to_bf16_bits(v[2 * e + 1])) << 16);
    *reinterpret_cast<uint4*>(static_cast<uint16_t*>(p) + i) = make_uint4(w[0], w[1], w[2], w[3]);
  } else if (VEC == 8) {
    *reinterpret_cast<float4*>(static_cast<float*>(p) + i) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(static_cast<float*>(p) + i + 4) = make_float4(v[4], v[5], v[6], v[7]);
  } else {
#pragma unroll
    for (int e = 0; e < VEC; ++e) g_store<kBf16>(p, i + e, v[e]);
  }
}

template <bool kBf16, int VEC>
__global__ __launch_bounds__(kNormThreads) void add_rms_norm_kernel(AddNormArgs a) {
  constexpr int STEPS = kNormMaxDim / (kNormThreads * VEC);
  __shared__ float part[kNormThreads / kWave];
  const int64_t base = (int64_t)blockIdx.x * a.dim;
  const int tid = threadIdx.x;
  float v[STEPS][VEC], wv[STEPS][VEC], cv[STEPS][VEC];
  const bool carry_read = a.carry_mode == 2 || a.carry_mode == 4;
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < STEPS; ++j) {
    const int c = (j * kNormThreads + tid) * VEC;
    if (c < a.dim) {
      load_vec<kBf16, VEC>(a.x, base + c, v[j]);
      // (what the second pass needs is requested now, so that it does not wait for memory again)
      load_vec<kBf16, VEC>(a.weight, c, wv[j]);
      if (carry_read) load_vec<kBf16, VEC>(a.carry, base + c, cv[j]);
      if (a.delta) {
        float d[VEC];
        load_vec<kBf16, VEC>(a.delta, base + c, d);
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[j][e] = g_round<kBf16>(v[j][e] + d[e]);
        store_vec<kBf16, VEC>(a.x, base + c, v[j]);
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) ss += v[j][e] * v[j][e];
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
  if ((tid & 63) == 0) part[tid >> 6] = ss;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int w = 0; w < kNormThreads / kWave; ++w) tot += part[w];
  const float r = rsqrtf(tot / (float)a.dim + a.eps);
#pragma unroll
  for (int j = 0; j < STEPS; ++j) {
    const int c = (j * kNormThreads + tid) * VEC;
    if (c < a.dim) {
      float h[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) h[e] = g_round<kBf16>(g_round<kBf16>(v[j][e] * r) * wv[j][e]);
      store_vec<kBf16, VEC>(a.out, base + c, h);
      if (a.carry_mode) {
        float cn[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          if (a.carry_mode <= 2) {
            const float add = g_round<kBf16>(h[e] / a.chunk);
            cn[e] = a.carry_mode == 1 ? add : g_round<kBf16>(cv[j][e] + add);
          } else {
            cn[e] = a.carry_mode == 3 ? h[e] : fmaxf(cv[j][e], h[e]);
          }
        }
        store_vec<kBf16, VEC>(a.carry, base + c, cn);
      }
    }
  }
}

// VEC consecutive columns per thread (16-byte loads and stores when the rows allow it, else 1)
template <bool kBf16, int VEC>
__global__ __launch_bounds__(256) void silu_mul_kernel(const void* __restrict__ gate_up, void* __restrict__ out, int64_t rows,
                                                        int inter) {
  const int per_row = inter / VEC;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * per_row) return;
  const int64_t r = i / per_row;
  const int c = (int)(i - r * per_row) * VEC;
  float g[VEC], u[VEC], y[VEC];
  load_vec<kBf16, VEC>(gate_up, r * 2 * inter + c, g);
  load_vec<kBf16, VEC>(gate_up, r * 2 * inter + inter + c, u);
#pragma unroll
  for (int e = 0; e < VEC; ++e) y[e] = g_round<kBf16>(g[e] / (1.f + expf(-g[e]))) * u[e];
  store_vec<kBf16, VEC>(out, r * inter + c, y);
}

// ---- y[r, n] = sum_k x[r, k] * w[n, k] for a few rows of x (the projections of a one-token step) --------------
// The weights are read once from HBM and nothing else is: one wavefront owns WR output columns, its lanes walk
// k in 16-byte pieces with UNROLL pieces of every weight row in flight, products and sums in fp32, one
// butterfly reduction per (column, x row) at the end.  Weight loads bypass the caches' retention (each byte is
// used once per step); x is re-read from cache by every wavefront.
// kGate: w holds the gate rows [0, N) and the up rows [N, 2N); the wavefront computes both for its columns and
// writes silu(gate) * up with the rounding points of the separate ops (projection, SiLU, product).
struct MatvecArgs {
  const void *w, *x;
  void* y;
  int64_t w_stride, x_stride, y_stride;  // elements
  int n_out, k;
};

constexpr int kMatvecWaves = 4;
constexpr int kMatvecUnroll = 4;

// a 16-byte piece of a weight row; the load is marked as a stream (no reuse)
__device__ __forceinline__ uint4 stream_load16(const unsigned char* p) {
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

template <bool kBf16>
__device__ __forceinline__ void unpack_piece(const uint4& u, float (&v)[8]) {
  // (fp32: only v[0..3] are used)
  if (kBf16) {
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[2 * e] = __uint_as_float(w[e] << 16);
      v[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
    }
  } else {
    v[0] = __uint_as_float(u.x); v[1] = __uint_as_float(u.y); v[2] = __uint_as_float(u.z); v[3] = __uint_as_float(u.w);
  }
}

template <bool kBf16, int XR, int WR, bool kGate>
__global__ __launch_bounds__(kMatvecWaves * kWave) void matvec_kernel(MatvecArgs a) {
  constexpr int E = kBf16 ? 8 : 4;       // elements per 16-byte piece
  constexpr int NW = kGate ? 2 * WR : WR;  // weight rows per wavefront
  constexpr int ES = kBf16 ? 2 : 4;      // bytes per element
  const int lane = lane_id();
  const int n0 = (blockIdx.x * kMatvecWaves + (threadIdx.x >> 6)) * WR;
  if (n0 >= a.n_out) return;
  const unsigned char* wrow[NW];
#pragma unroll
  for (int j = 0; j < NW; ++j) {
    // columns past the end repeat the last one (their results are not written)
    const int col = min(n0 + (j % WR), a.n_out - 1);
    const int64_t row = (kGate && j >= WR) ? (int64_t)a.n_out + col : col;
    wrow[j] = static_cast<const unsigned char*>(a.w) + row * a.w_stride * ES;
  }
  const unsigned char* xp = static_cast<const unsigned char*>(a.x);
  float acc[NW][XR];
#pragma unroll
  for (int j = 0; j < NW; ++j)
#pragma unroll
    for (int r = 0; r < XR; ++r) acc[j][r] = 0.f;

  const int pieces = a.k / E;
  auto step = [&](int p, const uint4 (&wv)[NW]) {
    float xv[XR][8];
#pragma unroll
    for (int r = 0; r < XR; ++r) {
      const uint4 u = *reinterpret_cast<const uint4*>(xp + (r * a.x_stride + (int64_t)p * E) * ES);
      unpack_piece<kBf16>(u, xv[r]);
    }
#pragma unroll
    for (int j = 0; j < NW; ++j) {
      float wf[8];
      unpack_piece<kBf16>(wv[j], wf);
#pragma unroll
      for (int r = 0; r < XR; ++r)
#pragma unroll
        for (int e = 0; e < E; ++e) acc[j][r] = fmaf(wf[e], xv[r][e], acc[j][r]);
    }
  };
  int p = lane;
  // batches of kMatvecUnroll pieces per weight row, then one of half that, then single pieces
  auto batch = [&](auto n_const) {
    constexpr int N = decltype(n_const)::value;
    uint4 wv[N][NW];
#pragma unroll
    for (int u = 0; u < N; ++u)
#pragma unroll
      for (int j = 0; j < NW; ++j) wv[u][j] = stream_load16(wrow[j] + (int64_t)(p + u * kWave) * 16);
#pragma unroll
    for (int u = 0; u < N; ++u) step(p + u * kWave, wv[u]);
    p += N * kWave;
  };
  while (p + (kMatvecUnroll - 1) * kWave < pieces) batch(std::integral_constant<int, kMatvecUnroll>{});
  if (p + (kMatvecUnroll / 2 - 1) * kWave < pieces) batch(std::integral_constant<int, kMatvecUnroll / 2>{});
  for (; p < pieces; p += kWave) {
    uint4 wv[NW];
#pragma unroll
    for (int j = 0; j < NW; ++j) wv[j] = stream_load16(wrow[j] + (int64_t)p * 16);
    step(p, wv);
  }
#pragma unroll
  for (int j = 0; j < NW; ++j)
#pragma unroll
    for (int r = 0; r < XR; ++r)
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) acc[j][r] += __shfl_xor(acc[j][r], o);
  if (lane == 0) {
#pragma unroll
    for (int j = 0; j < WR; ++j) {
      if (n0 + j >= a.n_out) break;
#pragma unroll
      for (int r = 0; r < XR; ++r) {
        float v = acc[j][r];
        if (kGate) {
          const float g = g_round<kBf16>(v), u = g_round<kBf16>(acc[j + WR][r]);
          v = g_round<kBf16>(g / (1.f + expf(-g))) * u;
        }
        g_store<kBf16>(a.y, r * a.y_stride + n0 + j, v);
      }
    }
  }
}

struct RopeAppendArgs {
  const void *q, *k, *v, *cos, *sin;
  void *q_out, *cache_k, *cache_v;
  uint8_t* valid;
  int32_t* pos;
  int64_t qs[3], ks[3], vs[3];  // strides (b, h, l) of q, k, v; last dim contiguous
  int64_t cs[2];                // strides (b, l) of cos / sin
  int64_t cache_s[3];           // strides (b, h, row) of cache_k / cache_v
  int64_t valid_s[2];           // strides (b, h) of valid / pos
  int Hq, Hkv, x_len, D;
  int64_t row0;
  int pos0;
  int64_t clear_row;  // >= 0: valid[b, h, clear_row] is set to 0 for every (b, h) (a row below row0)
};

// grid (x_len, Hq + 2 * Hkv, B); one thread per element of the head vector (D <= 256)
template <bool kBf16>
__global__ void rope_append_kernel(RopeAppendArgs a) {
#pragma clang fp contract(off)  // the two products and their sum round separately, as the torch ops do (fp32 too)
  const int l = blockIdx.x, hh = blockIdx.y, b = blockIdx.z;
  const int d = threadIdx.x;
  if (d >= a.D) return;
  const int half = a.D / 2;
  const int64_t cidx = b * a.cs[0] + l * a.cs[1];
  if (hh < a.Hq + a.Hkv) {
    const bool is_q = hh < a.Hq;
    const int h = is_q ? hh : hh - a.Hq;
    const void* src = is_q ? a.q : a.k;
    const int64_t* st = is_q ? a.qs : a.ks;
    const int64_t s0 = b * st[0] + h * st[1] + l * st[2];
    const float x = g_load<kBf16>(src, s0 + d);
    const float xr = d < half ? -g_load<kBf16>(src, s0 + d + half) : g_load<kBf16>(src, s0 + d - half);
    const float p1 = g_round<kBf16>(x * g_load<kBf16>(a.cos, cidx + d));
    const float p2 = g_round<kBf16>(xr * g_load<kBf16>(a.sin, cidx + d));
    const float y = p1 + p2;
    if (is_q) {
      g_store<kBf16>(a.q_out, (((int64_t)b * a.Hq + h) * a.x_len + l) * a.D + d, y);
    } else {
      g_store<kBf16>(a.cache_k, b * a.cache_s[0] + h * a.cache_s[1] + (a.row0 + l) * a.cache_s[2] + d, y);
      if (d == 0) {
        a.valid[b * a.valid_s[0] + h * a.valid_s[1] + a.row0 + l] = 1;
        if (a.pos) a.pos[b * a.valid_s[0] + h * a.valid_s[1] + a.row0 + l] = a.pos0 + l;
        if (l == 0 && a.clear_row >= 0) a.valid[b * a.valid_s[0] + h * a.valid_s[1] + a.clear_row] = 0;
      }
    }
  } else {
    const int h = hh - a.Hq - a.Hkv;
    const float x = g_load<kBf16>(a.v, b * a.vs[0] + h * a.vs[1] + l * a.vs[2] + d);
    g_store<kBf16>(a.cache_v, b * a.cache_s[0] + h * a.cache_s[1] + (a.row0 + l) * a.cache_s[2] + d, x);
  }
}

// ---- rotary embedding of q and k of a multi-token segment (no cache write) -------------------------------------
// One thread rotates VEC consecutive dims of the first half of a head vector and their partners in the second
// half (16-byte loads and stores); a block of 256 threads takes 256 / (D / (2 VEC)) head vectors, ordered
// (b, l, head) as the projection output lies in memory.  Same rounding points as rope_append_kernel.
struct RopeQkArgs {
  const void *q, *k, *cos, *sin;
  void *q_out, *k_out;
  int64_t qs[3], ks[3];  // strides (b, h, l) of q, k; last dim contiguous
  int64_t cs[2];         // strides (b, l) of cos / sin
  int Hq, Hkv, x_len, D;
  int64_t n_vec;         // head vectors in all: B * x_len * (Hq + Hkv)
};

template <bool kBf16>
__global__ __launch_bounds__(256) void rope_qk_kernel(RopeQkArgs a) {
#pragma clang fp contract(off)
  constexpr int VEC = kBf16 ? 8 : 4;
  const int tpv = a.D / (2 * VEC);  // threads per head vector
  const int64_t vec = (int64_t)blockIdx.x * (256 / tpv) + threadIdx.x / tpv;
  if (threadIdx.x >= (256 / tpv) * tpv || vec >= a.n_vec) return;
  const int d = (threadIdx.x % tpv) * VEC;
  const int half = a.D / 2;
  const int H = a.Hq + a.Hkv;
  const int hh = (int)(vec % H);
  const int64_t bl = vec / H;
  const int l = (int)(bl % a.x_len), b = (int)(bl / a.x_len);
  const bool is_q = hh < a.Hq;
  const int h = is_q ? hh : hh - a.Hq;
  const void* src = is_q ? a.q : a.k;
  const int64_t* st = is_q ? a.qs : a.ks;
  const int64_t s0 = b * st[0] + h * st[1] + l * st[2];
  const int64_t c0 = b * a.cs[0] + l * a.cs[1];
  float lo[VEC], hi[VEC], c_lo[VEC], c_hi[VEC], s_lo[VEC], s_hi[VEC], y_lo[VEC], y_hi[VEC];
  if (kBf16) {
    float t8[8];
    load_vec<true, 8>(src, s0 + d, t8);
    for (int e = 0; e < VEC; ++e) lo[e] = t8[e];
    load_vec<true, 8>(src, s0 + d + half, t8);
    for (int e = 0; e < VEC; ++e) hi[e] = t8[e];
    load_vec<true, 8>(a.cos, c0 + d, t8);
    for (int e = 0; e < VEC; ++e) c_lo[e] = t8[e];
    load_vec<true, 8>(a.cos, c0 + d + half, t8);
    for (int e = 0; e < VEC; ++e) c_hi[e] = t8[e];
    load_vec<true, 8>(a.sin, c0 + d, t8);
    for (int e = 0; e < VEC; ++e) s_lo[e] = t8[e];
    load_vec<true, 8>(a.sin, c0 + d + half, t8);
    for (int e = 0; e < VEC; ++e) s_hi[e] = t8[e];
  } else {
    const auto ld4 = [](const void* p, int64_t i, float (&v)[VEC]) {
      const float4 r = *reinterpret_cast<const float4*>(static_cast<const float*>(p) + i);
      v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
    };
    ld4(src, s0 + d, lo); ld4(src, s0 + d + half, hi);
    ld4(a.cos, c0 + d, c_lo); ld4(a.cos, c0 + d + half, c_hi);
    ld4(a.sin, c0 + d, s_lo); ld4(a.sin, c0 + d + half, s_hi);
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    y_lo[e] = g_round<kBf16>(lo[e] * c_lo[e]) + g_round<kBf16>(-hi[e] * s_lo[e]);
    y_hi[e] = g_round<kBf16>(hi[e] * c_hi[e]) + g_round<kBf16>(lo[e] * s_hi[e]);
  }
  void* dst = is_q ? a.q_out : a.k_out;
  const int64_t o0 = (((int64_t)b * (is_q ? a.Hq : a.Hkv) + h) * a.x_len + l) * a.D;
  if (kBf16) {
    float t8[8];
    for (int e = 0; e < VEC; ++e) t8[e] = y_lo[e];
    store_vec<true, 8>(dst, o0 + d, t8);
    for (int e = 0; e < VEC; ++e) t8[e] = y_hi[e];
    store_vec<true, 8>(dst, o0 + d + half, t8);
  } else {
    *reinterpret_cast<float4*>(static_cast<float*>(dst) + o0 + d) = make_float4(y_lo[0], y_lo[1], y_lo[2], y_lo[3]);
    *reinterpret_cast<float4*>(static_cast<float*>(dst) + o0 + d + half) = make_float4(y_hi[0], y_hi[1], y_hi[2], y_hi[3]);
  }
}

}  // namespace nats

using namespace nats;

extern "C" int nats_add_rms_norm(void* x, const void* delta, const void* weight, void* out, void* carry, int64_t rows,
                                 int64_t dim, float eps, int carry_mode, int64_t chunk_size, int dtype, void* stream) {
  NATS_REQUIRE(x && weight && out, NATS_ERR_NULL_POINTER, "nats_add_rms_norm: NULL pointer");
  NATS_REQUIRE(rows > 0 && dim > 0 && dim <= kNormMaxDim && rows <= 0x7fffffff, NATS_ERR_BAD_SHAPE,
               "nats_add_rms_norm: rows=%lld dim=%lld (dim <= %d)", (long long)rows, (long long)dim, kNormMaxDim);
  NATS_REQUIRE(dtype == NATS_DTYPE_BF16 || dtype == NATS_DTYPE_F32, NATS_ERR_BAD_DTYPE, "nats_add_rms_norm: dtype %d", dtype);
  NATS_REQUIRE(carry_mode >= 0 && carry_mode <= 4 && (carry_mode == 0 || (carry && chunk_size > 0)), NATS_ERR_BAD_SHAPE,
               "nats_add_rms_norm: carry_mode %d needs a carry buffer and a chunk size", carry_mode);
  AddNormArgs a{x, delta, weight, out, carry, (int)dim, carry_mode, eps, (float)chunk_size};
  hipStream_t st = static_cast<hipStream_t>(stream);
  auto aligned16 = [](const void* p) { return p == nullptr || reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = dim % 8 == 0 && aligned16(x) && aligned16(delta) && aligned16(weight) && aligned16(out) && aligned16(carry);
  const dim3 grid((unsigned)rows), block(kNormThreads);
  if (dtype == NATS_DTYPE_BF16) {
    if (vec) {
      hipLaunchKernelGGL((add_rms_norm_kernel<true, 8>), grid, block, 0, st, a);
    } else {
      hipLaunchKernelGGL((add_rms_norm_kernel<true, 1>), grid, block, 0, st, a);
    }
  } else {
    if (vec) {
      hipLaunchKernelGGL((add_rms_norm_kernel<false, 8>), grid, block, 0, st, a);
    } else {
      hipLaunchKernelGGL((add_rms_norm_kernel<false, 1>), grid, block, 0, st, a);
    }
  }
  NATS_CHECK_LAUNCH("add_rms_norm_kernel");
  return NATS_OK;
}

extern "C" int nats_silu_mul(const void* gate_up, void* out, int64_t rows, int64_t inter, int dtype, void* stream) {
  NATS_REQUIRE(gate_up && out, NATS_ERR_NULL_POINTER, "nats_silu_mul: NULL pointer");
  NATS_REQUIRE(rows > 0 && inter > 0 && inter <= 0x3fffffff && rows * inter <= (int64_t)0x7fffffff * 256, NATS_ERR_BAD_SHAPE,
               "nats_silu_mul: rows=%lld inter=%lld", (long long)rows, (long long)inter);
  NATS_REQUIRE(dtype == NATS_DTYPE_BF16 || dtype == NATS_DTYPE_F32, NATS_ERR_BAD_DTYPE, "nats_silu_mul: dtype %d", dtype);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool wide = inter % 8 == 0 && ((reinterpret_cast<uintptr_t>(gate_up) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
  const int64_t n_threads = wide ? rows * (inter / 8) : rows * inter;
  const unsigned blocks = (unsigned)((n_threads + 255) / 256);
  if (dtype == NATS_DTYPE_BF16) {
    if (wide) {
      hipLaunchKernelGGL((silu_mul_kernel<true, 8>), dim3(blocks), dim3(256), 0, st, gate_up, out, rows, (int)inter);
    } else {
      hipLaunchKernelGGL((silu_mul_kernel<true, 1>), dim3(blocks), dim3(256), 0, st, gate_up, out, rows, (int)inter);
    }
  } else {
    if (wide) {
      hipLaunchKernelGGL((silu_mul_kernel<false, 8>), dim3(blocks), dim3(256), 0, st, gate_up, out, rows, (int)inter);
    } else {
      hipLaunchKernelGGL((silu_mul_kernel<false, 1>), dim3(blocks), dim3(256), 0, st, gate_up, out, rows, (int)inter);
    }
  }
  NATS_CHECK_LAUNCH("silu_mul_kernel");
  return NATS_OK;
}

template <bool kBf16, int XR, bool kGate>
static void launch_matvec(const MatvecArgs& a, hipStream_t st) {
  // wide outputs: two columns per wavefront (more bytes in flight per lane); narrow ones keep one column per
  // wavefront so that every CU has wavefronts
  const bool two = !kGate && a.n_out >= 8192;
  const int per_wave = two ? 2 : 1;
  const unsigned blocks = (unsigned)((a.n_out + per_wave * kMatvecWaves - 1) / (per_wave * kMatvecWaves));
  if (two) {
    hipLaunchKernelGGL((matvec_kernel<kBf16, XR, 2, kGate>), dim3(blocks), dim3(kMatvecWaves * kWave), 0, st, a);
  } else {
    hipLaunchKernelGGL((matvec_kernel<kBf16, XR, 1, kGate>), dim3(blocks), dim3(kMatvecWaves * kWave), 0, st, a);
  }
}

template <bool kBf16, bool kGate>
static void launch_matvec_rows(const MatvecArgs& a, int x_rows, hipStream_t st) {
  switch (x_rows) {
    case 1: launch_matvec<kBf16, 1, kGate>(a, st); break;
    case 2: launch_matvec<kBf16, 2, kGate>(a, st); break;
    case 3: launch_matvec<kBf16, 3, kGate>(a, st); break;
    default: launch_matvec<kBf16, 4, kGate>(a, st); break;
  }
}

extern "C" int nats_matvec(const void* w, const void* x, void* y, int64_t x_rows, int64_t n_out, int64_t k,
                           int64_t w_stride, int64_t x_stride, int64_t y_stride, int gate, int dtype, void* stream) {
  NATS_REQUIRE(w && x && y, NATS_ERR_NULL_POINTER, "nats_matvec: NULL pointer");
  NATS_REQUIRE(dtype == NATS_DTYPE_BF16 || dtype == NATS_DTYPE_F32, NATS_ERR_BAD_DTYPE, "nats_matvec: dtype %d", dtype);
  const int64_t e = dtype == NATS_DTYPE_BF16 ? 8 : 4;
  NATS_REQUIRE(x_rows >= 1 && x_rows <= 4, NATS_ERR_UNSUPPORTED, "nats_matvec: %lld rows of x (1..4)", (long long)x_rows);
  NATS_REQUIRE(n_out > 0 && n_out <= 0x3fffffff && k > 0 && k <= 0x3fffffff, NATS_ERR_BAD_SHAPE,
               "nats_matvec: n_out=%lld k=%lld", (long long)n_out, (long long)k);
  NATS_REQUIRE(k % e == 0 && w_stride % e == 0 && x_stride % e == 0 && w_stride >= k && x_stride >= k && y_stride >= n_out,
               NATS_ERR_BAD_SHAPE, "nats_matvec: k=%lld and the strides of w (%lld) and x (%lld) must be multiples of %lld",
               (long long)k, (long long)w_stride, (long long)x_stride, (long long)e);
  NATS_REQUIRE((reinterpret_cast<uintptr_t>(w) & 15) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0, NATS_ERR_BAD_SHAPE,
               "nats_matvec: w and x must be 16-byte aligned");
  MatvecArgs a{};
  a.w = w; a.x = x; a.y = y;
  a.w_stride = w_stride; a.x_stride = x_stride; a.y_stride = y_stride;
  a.n_out = (int)n_out; a.k = (int)k;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == NATS_DTYPE_BF16) {
    if (gate) launch_matvec_rows<true, true>(a, (int)x_rows, st); else launch_matvec_rows<true, false>(a, (int)x_rows, st);
  } else {
    if (gate) launch_matvec_rows<false, true>(a, (int)x_rows, st); else launch_matvec_rows<false, false>(a, (int)x_rows, st);
  }
  NATS_CHECK_LAUNCH("matvec_kernel");
  return NATS_OK;
}

extern "C" int nats_rope_append(const void* q, const void* k, const void* v, const void* cos, const void* sin, void* q_out,
                                void* cache_k, void* cache_v, uint8_t* valid, int32_t* pos, int64_t B, int64_t H_q,
                                int64_t H_kv, int64_t x_len, int64_t D, int64_t row0, int64_t n_alloc, int64_t pos0,
                                int64_t clear_row, const int64_t* q_strides, const int64_t* k_strides,
                                const int64_t* v_strides, const int64_t* cos_strides, const int64_t* cache_strides,
                                const int64_t* valid_strides, int dtype, void* stream) {
  NATS_REQUIRE(q && k && v && cos && sin && q_out && cache_k && cache_v && valid, NATS_ERR_NULL_POINTER,
               "nats_rope_append: NULL pointer");
  NATS_REQUIRE(clear_row < row0, NATS_ERR_BAD_SHAPE, "nats_rope_append: clear_row=%lld is not below row0=%lld",
               (long long)clear_row, (long long)row0);
  NATS_REQUIRE(q_strides && k_strides && v_strides && cos_strides && cache_strides && valid_strides, NATS_ERR_NULL_POINTER,
               "nats_rope_append: NULL stride array");
  NATS_REQUIRE(B > 0 && H_q > 0 && H_kv > 0 && x_len > 0 && B <= 65535 && H_q + 2 * H_kv <= 65535, NATS_ERR_BAD_SHAPE,
               "nats_rope_append: B=%lld H_q=%lld H_kv=%lld x_len=%lld", (long long)B, (long long)H_q, (long long)H_kv,
               (long long)x_len);
  NATS_REQUIRE(D > 0 && D % 2 == 0 && D <= 256, NATS_ERR_UNSUPPORTED, "nats_rope_append: head_dim %lld", (long long)D);
  NATS_REQUIRE(row0 >= 0 && row0 + x_len <= n_alloc, NATS_ERR_BAD_SHAPE, "nats_rope_append: rows [%lld, %lld) of %lld",
               (long long)row0, (long long)(row0 + x_len), (long long)n_alloc);
  NATS_REQUIRE(dtype == NATS_DTYPE_BF16 || dtype == NATS_DTYPE_F32, NATS_ERR_BAD_DTYPE, "nats_rope_append: dtype %d", dtype);
  RopeAppendArgs a{};
  a.q = q; a.k = k; a.v = v; a.cos = cos; a.sin = sin;
  a.q_out = q_out; a.cache_k = cache_k; a.cache_v = cache_v; a.valid = valid; a.pos = pos;
  for (int i = 0; i < 3; ++i) {
    a.qs[i] = q_strides[i]; a.ks[i] = k_strides[i]; a.vs[i] = v_strides[i]; a.cache_s[i] = cache_strides[i];
  }
  for (int i = 0; i < 2; ++i) {
    a.cs[i] = cos_strides[i]; a.valid_s[i] = valid_strides[i];
  }
  a.Hq = (int)H_q; a.Hkv = (int)H_kv; a.x_len = (int)x_len; a.D = (int)D;
  a.row0 = row0; a.pos0 = (int)pos0;
  a.clear_row = clear_row;
  hipStream_t st = static_cast<hipStream_t>(stream);
  dim3 grid((unsigned)x_len, (unsigned)(H_q + 2 * H_kv), (unsigned)B);
  const unsigned threads = (unsigned)((D + 63) / 64 * 64);
  if (dtype == NATS_DTYPE_BF16) {
    hipLaunchKernelGGL(rope_append_kernel<true>, grid, dim3(threads), 0, st, a);
  } else {
    hipLaunchKernelGGL(rope_append_kernel<false>, grid, dim3(threads), 0, st, a);
  }
  NATS_CHECK_LAUNCH("rope_append_kernel");
  return NATS_OK;
}

extern "C" int nats_rope_qk(const void* q, const void* k, const void* cos, const void* sin, void* q_out, void* k_out, int64_t B,
                            int64_t H_q, int64_t H_kv, int64_t x_len, int64_t D, const int64_t* q_strides,
                            const int64_t* k_strides, const int64_t* cos_strides, int dtype, void* stream) {
  NATS_REQUIRE(q && k && cos && sin && q_out && k_out && q_strides && k_strides && cos_strides, NATS_ERR_NULL_POINTER,
               "nats_rope_qk: NULL pointer");
  NATS_REQUIRE(dtype == NATS_DTYPE_BF16 || dtype == NATS_DTYPE_F32, NATS_ERR_BAD_DTYPE, "nats_rope_qk: dtype %d", dtype);
  const int64_t vec = dtype == NATS_DTYPE_BF16 ? 8 : 4;
  NATS_REQUIRE(B > 0 && H_q > 0 && H_kv > 0 && x_len > 0 && B * x_len * (H_q + H_kv) < (int64_t(1) << 40), NATS_ERR_BAD_SHAPE,
               "nats_rope_qk: B=%lld H_q=%lld H_kv=%lld x_len=%lld", (long long)B, (long long)H_q, (long long)H_kv,
               (long long)x_len);
  NATS_REQUIRE(D > 0 && D % (2 * vec) == 0 && D <= 512, NATS_ERR_UNSUPPORTED, "nats_rope_qk: head_dim %lld", (long long)D);
  bool aligned = ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(cos) |
                   reinterpret_cast<uintptr_t>(sin) | reinterpret_cast<uintptr_t>(q_out) | reinterpret_cast<uintptr_t>(k_out)) & 15) == 0;
  for (int i = 0; i < 3; ++i) aligned = aligned && q_strides[i] % vec == 0 && k_strides[i] % vec == 0;
  for (int i = 0; i < 2; ++i) aligned = aligned && cos_strides[i] % vec == 0;
  NATS_REQUIRE(aligned, NATS_ERR_BAD_SHAPE, "nats_rope_qk: rows must be 16-byte aligned");
  RopeQkArgs a{};
  a.q = q; a.k = k; a.cos = cos; a.sin = sin; a.q_out = q_out; a.k_out = k_out;
  for (int i = 0; i < 3; ++i) {
    a.qs[i] = q_strides[i]; a.ks[i] = k_strides[i];
  }
  a.cs[0] = cos_strides[0]; a.cs[1] = cos_strides[1];
  a.Hq = (int)H_q; a.Hkv = (int)H_kv; a.x_len = (int)x_len; a.D = (int)D;
  a.n_vec = B * x_len * (H_q + H_kv);
  const int tpv = (int)(D / (2 * vec));
  const int64_t per_block = 256 / tpv;
  const int64_t blocks = (a.n_vec + per_block - 1) / per_block;
  NATS_REQUIRE(blocks < (int64_t(1) << 31), NATS_ERR_BAD_SHAPE, "nats_rope_qk: grid too large");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == NATS_DTYPE_BF16) {
    hipLaunchKernelGGL(rope_qk_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, st, a);
  } else {
    hipLaunchKernelGGL(rope_qk_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, st, a);
  }
  NATS_CHECK_LAUNCH("rope_qk_kernel");
  return NATS_OK;
}
