// Fused role step: chunk pooling of the hidden states, the role projection, the bias on the global option,
// the argmax with its forced globals and (through role_scan_kernel) the next-global scan, in one entry point.
//
// Follows NAtSCache.update_nats_cached_x_across_chunk (components/cache/dyn_cache.py:130-171), the pooling of
// chunk_utils.py:13-62, proj_layer + _sample_for_token_info_values_inference
// (models/transformer/attention/nats_chunk_attention.py:64-95, nats_attention.py:96-109) and
// generate_hard_seq_masks' index scan (components/masks/utils.py:85-87).
//
// Rounding points are those of the torch ops the reference runs: the pooled statistic is rounded to the
// input dtype, the logits are accumulated in fp32 and rounded to the input dtype, the bias is added in that
// dtype.  (fp32 summation order differs from a library GEMM, so logits agree with it to rounding, not bit
// for bit; the roles are the exact argmax of the logits this kernel writes.)
#include "nats_common.h"

namespace nats {

int launch_role_scan(const uint8_t* roles, int64_t n_streams, int64_t S, int64_t W, int64_t C, int64_t* end_idx,
                     int32_t* vis_lim, int32_t* first_global, hipStream_t st);

struct RoleStepArgs {
  const void* x;        // [B, L, dim]
  const void* carry_in; // [B, dim] or null
  const void* weight;   // [H_kv * 3, dim]
  uint8_t* roles;       // [B, H_kv, S]
  void* one_hot;        // [B, H_kv, S, 3] or null
  void* logits;         // [B, S, H_kv, 3] or null
  void* carry_out;      // [B, dim] or null
  int64_t xs_b, xs_l;
  int B, L, dim, Hkv, C, S, pre_fill, pad;
  int merge_max, first_g;
  int hpb;  // role streams (kv heads) whose logits one workgroup computes; blockIdx.z counts groups of them
  int64_t roles_hs;  // entries between the roles of two consecutive (b, kv head) streams (S when they are contiguous)
  float bias;
};

template <bool kBf16>
__device__ __forceinline__ float load_elem(const void* p, int64_t i) {
  if (kBf16) return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
  return static_cast<const float*>(p)[i];
}
template <bool kBf16>
__device__ __forceinline__ float round_elem(float v) {
  return kBf16 ? bf16_bits_to_f32(f32_to_bf16_bits(v)) : v;
}
template <bool kBf16>
__device__ __forceinline__ void store_elem(void* p, int64_t i, float v) {
  if (kBf16) {
    static_cast<uint16_t*>(p)[i] = f32_to_bf16_bits(v);
  } else {
    static_cast<float*>(p)[i] = v;
  }
}

// One workgroup per (chunk, batch row, group of hpb role streams).  Block (0, b) also serves the case without a
// complete chunk (S == 0), where only the running statistic is updated.  With few chunks (the token that closes a
// chunk while decoding, every token of a per-token cache) the role streams are spread over workgroups, each of which
// pools the chunk for itself and projects it onto its own streams' three weight rows: the 24 dot products of a
// Llama-3-8B layer then run side by side instead of six per wavefront one after the other.  VEC consecutive columns
// per thread (16-byte loads when the rows allow it, else 1).
template <bool kBf16, int VEC>
__global__ __launch_bounds__(256) void role_step_kernel(RoleStepArgs a) {
  extern __shared__ float pooled[];  // [dim] statistic of this chunk, then [Hkv * 3] logits behind it
  float* logit_s = pooled + a.dim;
  const int s = blockIdx.x, b = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float inv_c = 1.f / float(a.C);

  // tokens of x that belong to chunk s
  const int t0 = max(s * a.C - a.pre_fill, 0);
  const int t1 = min((s + 1) * a.C - a.pre_fill, a.L);
  const bool with_carry = s == 0 && a.pre_fill > 0 && a.carry_in != nullptr;
  const bool padded = a.S > 0 && s == a.S - 1 && a.pad != 0;  // zero rows take part in the statistic
  const char* xb = static_cast<const char*>(a.x);
  constexpr int esz = kBf16 ? 2 : 4;
  for (int d = tid * VEC; d < a.dim; d += 256 * VEC) {
    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = a.merge_max ? -INFINITY : 0.f;
    // kAhead rows are requested before the first of them is used (the sums keep the order of the rows)
    auto load_row = [&](int t, float (&e)[VEC]) {
      const char* row = xb + (b * a.xs_b + t * a.xs_l + d) * esz;
      if (VEC == 1) {
        e[0] = load_elem<kBf16>(row, 0);
      } else if (kBf16) {
        uint4 raw = *reinterpret_cast<const uint4*>(row);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int v = 0; v < VEC; ++v) e[v] = bf16_bits_to_f32(uint16_t(w[v >> 1] >> ((v & 1) * 16)));
      } else {
        float4 raw = *reinterpret_cast<const float4*>(row);
        const float w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int v = 0; v < VEC; ++v) e[v] = w[v];
      }
    };
    constexpr int kAhead = 8;
    int t = t0;
    for (; t + kAhead <= t1; t += kAhead) {
      float e[kAhead][VEC];
#pragma unroll
      for (int u = 0; u < kAhead; ++u) load_row(t + u, e[u]);
#pragma unroll
      for (int u = 0; u < kAhead; ++u)
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] = a.merge_max ? fmaxf(acc[v], e[u][v]) : acc[v] + e[u][v];
    }
    for (; t < t1; ++t) {
      float e[VEC];
      load_row(t, e);
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc[v] = a.merge_max ? fmaxf(acc[v], e[v]) : acc[v] + e[v];
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      float stat, tail_max = acc[v];
      if (!a.merge_max) {
        stat = round_elem<kBf16>(acc[v] * inv_c);  // power-of-two C: x / C is exact, so both torch forms agree
        if (with_carry) stat = round_elem<kBf16>(load_elem<kBf16>(a.carry_in, (int64_t)b * a.dim + d + v) + stat);
      } else {
        stat = acc[v];
        if (with_carry) stat = fmaxf(stat, load_elem<kBf16>(a.carry_in, (int64_t)b * a.dim + d + v));
        if (padded) stat = fmaxf(stat, 0.f);
      }
      pooled[d + v] = stat;
      // the statistic carried to the next call: the open last chunk, or everything so far when no chunk completes
      if (a.carry_out && (a.S == 0 || padded) && blockIdx.z == 0) {
        store_elem<kBf16>(a.carry_out, (int64_t)b * a.dim + d + v, a.merge_max ? (a.S == 0 ? stat : tail_max) : stat);
      }
    }
  }
  if (a.S == 0) return;
  __syncthreads();

  // logits[o] = sum_d pooled[d] * W[o][d]; wavefront w takes this workgroup's outputs w, w + 4, ...
  const int h0 = blockIdx.z * a.hpb, h1 = min(h0 + a.hpb, a.Hkv);
  const int n_out = h1 * 3;
  for (int o = h0 * 3 + wave; o < n_out; o += 4) {
    float acc = 0.f;
    if (VEC > 1) {
      // VEC consecutive weights per lane and step (one 16-byte load)
      const char* wrow = static_cast<const char*>(a.weight) + (int64_t)o * a.dim * esz;
      for (int d = lane * VEC; d < a.dim; d += 64 * VEC) {
        float w[VEC];
        if (kBf16) {
          const uint4 raw = *reinterpret_cast<const uint4*>(wrow + d * 2);
          const uint32_t u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
          for (int v = 0; v < VEC; ++v) w[v] = bf16_bits_to_f32(uint16_t(u[(v >> 1) & 3] >> ((v & 1) * 16)));
        } else {
          const float4 raw = *reinterpret_cast<const float4*>(wrow + d * 4);
          const float f[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
          for (int v = 0; v < VEC; ++v) w[v] = f[v & 3];
        }
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc = fmaf(pooled[d + v], w[v], acc);
      }
    } else {
      for (int d = lane; d < a.dim; d += 64) acc = fmaf(pooled[d], load_elem<kBf16>(a.weight, (int64_t)o * a.dim + d), acc);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) acc += __shfl_xor(acc, off);
    if (lane == 0) logit_s[o] = round_elem<kBf16>(acc);
  }
  __syncthreads();
  if (tid < h1 - h0) {
    const int h = h0 + tid;
    float x0 = logit_s[h * 3 + 0], x1 = logit_s[h * 3 + 1], x2 = logit_s[h * 3 + 2];
    if (a.logits) {
      int64_t base = (((int64_t)b * a.S + s) * a.Hkv + h) * 3;
      store_elem<kBf16>(a.logits, base + 0, x0);
      store_elem<kBf16>(a.logits, base + 1, x1);
      store_elem<kBf16>(a.logits, base + 2, x2);
    }
    x0 = round_elem<kBf16>(x0 + a.bias);
    int arg = 0;
    float best = x0;
    if (x1 > best) {
      best = x1;
      arg = 1;
    }
    if (x2 > best) arg = 2;
    if (a.first_g && s == 0) arg = NATS_ROLE_GLOBAL;
    if (a.pad != 0 && s == a.S - 1) arg = NATS_ROLE_GLOBAL;
    int64_t idx = ((int64_t)b * a.Hkv + h) * a.S + s;
    a.roles[((int64_t)b * a.Hkv + h) * a.roles_hs + s] = uint8_t(arg);
    if (a.one_hot) {
      store_elem<kBf16>(a.one_hot, idx * 3 + 0, arg == 0 ? 1.f : 0.f);
      store_elem<kBf16>(a.one_hot, idx * 3 + 1, arg == 1 ? 1.f : 0.f);
      store_elem<kBf16>(a.one_hot, idx * 3 + 2, arg == 2 ? 1.f : 0.f);
    }
  }
}

}  // namespace nats

using namespace nats;

extern "C" int nats_role_step(const void* x, const void* carry_in, const void* weight, int dtype, int64_t B, int64_t L,
                              int64_t dim, int64_t H_kv, int64_t C, int64_t W, int64_t pre_fill, int merge_max,
                              float global_bias, int force_first_global, const int64_t* x_strides, uint8_t* roles,
                              int64_t roles_head_stride, void* one_hot, void* logits, void* carry_out, int64_t* end_idx,
                              int32_t* vis_lim, void* stream) {
  const char* who = "nats_role_step";
  NATS_REQUIRE(x && weight && x_strides, NATS_ERR_NULL_POINTER, "%s: x, weight and x_strides must not be NULL", who);
  NATS_REQUIRE(B > 0 && L > 0 && dim > 0 && H_kv > 0 && B <= 65535, NATS_ERR_BAD_SHAPE, "%s: B=%lld L=%lld dim=%lld H_kv=%lld",
               who, (long long)B, (long long)L, (long long)dim, (long long)H_kv);
  NATS_REQUIRE(dtype == NATS_DTYPE_BF16 || dtype == NATS_DTYPE_F32, NATS_ERR_BAD_DTYPE, "%s: dtype %d", who, dtype);
  NATS_REQUIRE(is_pow2(C), NATS_ERR_UNSUPPORTED, "%s: chunk size %lld is not a power of two", who, (long long)C);
  NATS_REQUIRE(W >= 0 && W % C == 0, NATS_ERR_BAD_SHAPE, "%s: window %lld is not a multiple of chunk size %lld", who,
               (long long)W, (long long)C);
  NATS_REQUIRE(pre_fill >= 0 && pre_fill < C, NATS_ERR_BAD_SHAPE, "%s: pre_fill=%lld outside [0, %lld)", who,
               (long long)pre_fill, (long long)C);
  NATS_REQUIRE(pre_fill == 0 || carry_in, NATS_ERR_NULL_POINTER, "%s: an open chunk needs its running statistic", who);
  NATS_REQUIRE(H_kv <= 256 && (dim + 3 * H_kv) * sizeof(float) <= 160 * 1024, NATS_ERR_UNSUPPORTED,
               "%s: dim=%lld with %lld role streams does not fit the kernel", who, (long long)dim, (long long)H_kv);
  const int64_t total = pre_fill + L;
  const int64_t S = total < C ? 0 : (total + C - 1) / C;
  const int64_t pad = S == 0 ? 0 : S * C - total;
  NATS_REQUIRE(S == 0 || roles, NATS_ERR_NULL_POINTER, "%s: roles must not be NULL when a chunk completes", who);
  NATS_REQUIRE(S <= (int64_t(1) << 30), NATS_ERR_BAD_SHAPE, "%s: too many chunks", who);
  NATS_REQUIRE((S > 0 && pad == 0) || carry_out, NATS_ERR_NULL_POINTER, "%s: the open chunk's statistic needs carry_out", who);

  NATS_REQUIRE(roles_head_stride == 0 || (roles_head_stride >= S && !end_idx && !vis_lim), NATS_ERR_BAD_SHAPE,
               "%s: roles_head_stride=%lld (0 or at least the %lld chunks; the index scan takes contiguous roles)", who,
               (long long)roles_head_stride, (long long)S);
  RoleStepArgs a;
  a.roles_hs = roles_head_stride ? roles_head_stride : S;
  a.x = x; a.carry_in = carry_in; a.weight = weight; a.roles = roles; a.one_hot = one_hot; a.logits = logits;
  a.carry_out = carry_out;
  a.xs_b = x_strides[0]; a.xs_l = x_strides[1];
  a.B = (int)B; a.L = (int)L; a.dim = (int)dim; a.Hkv = (int)H_kv; a.C = (int)C; a.S = (int)S;
  a.pre_fill = (int)pre_fill; a.pad = (int)pad;
  a.merge_max = merge_max; a.first_g = force_first_global; a.bias = global_bias;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const size_t smem = (size_t)(dim + 3 * H_kv) * sizeof(float);
  // few chunks: a workgroup per role stream, so that the projection's rows are read side by side
  a.hpb = (S > 0 && S * B <= 32) ? 1 : (int)H_kv;
  dim3 grid((unsigned)(S > 0 ? S : 1), (unsigned)B, (unsigned)((H_kv + a.hpb - 1) / a.hpb));
  auto launch = [&](auto kernel) -> int {
    if (smem > 64 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
      if (e != hipSuccess) return fail(NATS_ERR_LAUNCH, "%s: hipFuncSetAttribute(%zu bytes of LDS): %s", who, smem, hipGetErrorString(e));
    }
    hipLaunchKernelGGL(kernel, grid, dim3(256), smem, st, a);
    return NATS_OK;
  };
  // 16-byte loads of x and of the projection weights when every row allows them
  const int vec = dtype == NATS_DTYPE_BF16 ? 8 : 4;
  const bool wide = dim % vec == 0 && x_strides[0] % vec == 0 && x_strides[1] % vec == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(weight) % 16 == 0;
  int rc;
  if (dtype == NATS_DTYPE_BF16) {
    rc = wide ? launch(role_step_kernel<true, 8>) : launch(role_step_kernel<true, 1>);
  } else {
    rc = wide ? launch(role_step_kernel<false, 4>) : launch(role_step_kernel<false, 1>);
  }
  if (rc) return rc;
  NATS_CHECK_LAUNCH("role_step_kernel");
  if (S > 0 && (end_idx || vis_lim)) return launch_role_scan(roles, B * H_kv, S, W, C, end_idx, vis_lim, nullptr, st);
  return NATS_OK;
}
