// Role assignment, next-global scan, and the debug outputs (token mask, tile map) derived from them.
#include "nats_common.h"

namespace nats {

static thread_local char g_error[512] = "";
char* error_buffer() { return g_error; }
int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

// ---------------------------------------------------------------------------------------------------
// logits [B, S, H, 3] -> roles [B, H, S] (+ one-hot [B, H, S, 3])
// Follows models/transformer/attention/nats_attention.py:99-107: bias on option 0 in the logits' dtype,
// first maximal option, slot 0 forced global inside the sink chunk; nats_chunk_attention.py:92-94: an
// open last chunk is forced global.
// ---------------------------------------------------------------------------------------------------
template <bool kBf16>
__global__ void roles_kernel(const void* __restrict__ logits, int64_t B, int64_t S, int64_t H, float bias, int first_g,
                             int last_g, uint8_t* __restrict__ roles, void* __restrict__ one_hot) {
  int64_t idx = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;  // over (b, h, s), s fastest: coalesced role writes
  int64_t total = B * H * S;
  if (idx >= total) return;
  int64_t s = idx % S;
  int64_t h = (idx / S) % H;
  int64_t b = idx / (S * H);
  int64_t in = ((b * S + s) * H + h) * 3;
  float x0, x1, x2;
  if (kBf16) {
    const uint16_t* p = static_cast<const uint16_t*>(logits) + in;
    // the bias add is a bf16 op in the reference: fp32 add, rounded back to bf16
    x0 = bf16_bits_to_f32(f32_to_bf16_bits(bf16_bits_to_f32(p[0]) + bias));
    x1 = bf16_bits_to_f32(p[1]);
    x2 = bf16_bits_to_f32(p[2]);
  } else {
    const float* p = static_cast<const float*>(logits) + in;
    x0 = p[0] + bias;
    x1 = p[1];
    x2 = p[2];
  }
  int arg = 0;
  float best = x0;
  if (x1 > best) {
    best = x1;
    arg = 1;
  }
  if (x2 > best) {
    arg = 2;
  }
  if (first_g && s == 0) arg = NATS_ROLE_GLOBAL;
  if (last_g && s == S - 1) arg = NATS_ROLE_GLOBAL;
  roles[idx] = uint8_t(arg);
  if (one_hot) {
    if (kBf16) {
      uint16_t* o = static_cast<uint16_t*>(one_hot) + idx * 3;
      o[0] = arg == 0 ? 0x3f80 : 0;
      o[1] = arg == 1 ? 0x3f80 : 0;
      o[2] = arg == 2 ? 0x3f80 : 0;
    } else {
      float* o = static_cast<float*>(one_hot) + idx * 3;
      o[0] = arg == 0 ? 1.f : 0.f;
      o[1] = arg == 1 ? 1.f : 0.f;
      o[2] = arg == 2 ? 1.f : 0.f;
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// One wavefront per (b, h): reverse scan in blocks of 64 slots with a ballot per block.
// end_idx[n] = first global slot >= n, the last slot counting as global (components/masks/utils.py:85-87).
// vis_lim[n] = last query slot that sees key slot n:
//   global -> INT32_MAX, sliding window -> n + W / C, local -> end_idx[n]
// (components/masks/utils.py:92 and components/cache/nats_chunk_layer_cache.py:603-611).
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void role_scan_kernel(const uint8_t* __restrict__ roles, int64_t S, int32_t wc,
                                                      int64_t* __restrict__ end_idx, int32_t* __restrict__ vis_lim) {
  const int64_t stream = blockIdx.x;
  const uint8_t* r = roles + stream * S;
  const int lane = lane_id();
  int64_t carry = S - 1;
  for (int64_t base = ((S - 1) / kWave) * kWave; base >= 0; base -= kWave) {
    int64_t n = base + lane;
    bool in = n < S;
    uint8_t role = in ? r[n] : uint8_t(NATS_ROLE_LOCAL);
    bool is_g = in && (role == NATS_ROLE_GLOBAL || n == S - 1);
    uint64_t bits = __ballot(is_g);
    uint64_t ahead = bits >> lane;  // bit 0 = this slot
    int64_t g = ahead ? n + __builtin_ctzll(ahead) : carry;
    if (in) {
      if (end_idx) end_idx[stream * S + n] = g;
      if (vis_lim) {
        int32_t lim;
        if (role == NATS_ROLE_GLOBAL) {
          lim = kLimGlobal;
        } else if (role == NATS_ROLE_SW) {
          lim = int32_t(n) + wc;
        } else {
          lim = int32_t(g);
        }
        vis_lim[stream * S + n] = lim;
      }
    }
    if (bits) carry = base + __builtin_ctzll(bits);
  }
}

// Per 64-key tile: the largest and the smallest vis_lim over the role slots the tile touches.
// tile_lim[stream][t] = {max, min}.  A query tile whose first slot is m0 must load key tile t iff
// max >= m0; every score of the pair is unmasked iff t lies strictly below the query tile and min >= the
// query tile's last slot.
__global__ void tile_lim_kernel(const int32_t* __restrict__ vis_lim, int64_t S, int64_t T, int c_shift,
                                int2* __restrict__ tile_lim) {
  int64_t idx = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  int64_t stream = blockIdx.y;
  if (idx >= T) return;
  int64_t n0 = (idx * kTile) >> c_shift;
  int64_t n1 = ((idx * kTile + kTile - 1) >> c_shift);
  if (n1 > S - 1) n1 = S - 1;
  int32_t mx = -1, mn = kLimGlobal;
  for (int64_t n = n0; n <= n1; ++n) {
    int32_t v = vis_lim[stream * S + n];
    mx = v > mx ? v : mx;
    mn = v < mn ? v : mn;
  }
  tile_lim[stream * T + idx] = make_int2(mx, mn);
}

// token-level mask, one thread per (query, key) pair
__global__ void mask_kernel(const int32_t* __restrict__ vis_lim, int64_t S, int64_t L, int c_shift,
                            uint8_t* __restrict__ mask) {
  int64_t n = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  int64_t m = blockIdx.y;
  int64_t stream = blockIdx.z;
  if (n >= L) return;
  bool vis = n <= m && (m >> c_shift) <= int64_t(vis_lim[stream * S + (n >> c_shift)]);
  mask[(stream * L + m) * L + n] = vis ? 1 : 0;
}

__global__ void tile_map_kernel(const int2* __restrict__ tile_lim, int64_t T, int c_shift, uint8_t* __restrict__ tiles) {
  int64_t kt = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  int64_t qt = blockIdx.y;
  int64_t stream = blockIdx.z;
  if (kt >= T) return;
  int64_t m0 = (qt * kTile) >> c_shift;
  bool visit = kt <= qt && int64_t(tile_lim[stream * T + kt].x) >= m0;
  tiles[(stream * T + qt) * T + kt] = visit ? 1 : 0;
}

int launch_role_scan(const uint8_t* roles, int64_t n_streams, int64_t S, int64_t W, int64_t C, int64_t* end_idx,
                     int32_t* vis_lim, hipStream_t st) {
  hipLaunchKernelGGL(role_scan_kernel, dim3((unsigned)n_streams), dim3(kWave), 0, st, roles, S, int32_t(W / C), end_idx,
                     vis_lim);
  NATS_CHECK_LAUNCH("role_scan_kernel");
  return NATS_OK;
}

int launch_tile_lim(const int32_t* vis_lim, int64_t n_streams, int64_t S, int64_t T, int64_t C, int2* tile_lim,
                    hipStream_t st) {
  dim3 grid((unsigned)((T + 255) / 256), (unsigned)n_streams);
  hipLaunchKernelGGL(tile_lim_kernel, grid, dim3(256), 0, st, vis_lim, S, T, ilog2(C), tile_lim);
  NATS_CHECK_LAUNCH("tile_lim_kernel");
  return NATS_OK;
}

}  // namespace nats

using namespace nats;

extern "C" int nats_abi_version(void) { return NATS_ABI_VERSION; }
extern "C" const char* nats_last_error(void) { return error_buffer(); }

extern "C" int nats_roles_from_logits(const void* logits, int dtype, int64_t B, int64_t S, int64_t H_kv,
                                      float global_bias, int force_first_global, int force_last_global,
                                      uint8_t* roles, void* one_hot, void* stream) {
  NATS_REQUIRE(logits && roles, NATS_ERR_NULL_POINTER, "nats_roles_from_logits: logits and roles must not be NULL");
  NATS_REQUIRE(B > 0 && S > 0 && H_kv > 0, NATS_ERR_BAD_SHAPE, "nats_roles_from_logits: B=%lld S=%lld H_kv=%lld",
               (long long)B, (long long)S, (long long)H_kv);
  NATS_REQUIRE(dtype == NATS_DTYPE_BF16 || dtype == NATS_DTYPE_F32, NATS_ERR_BAD_DTYPE,
               "nats_roles_from_logits: dtype %d", dtype);
  int64_t total = B * S * H_kv;
  dim3 grid((unsigned)((total + 255) / 256));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == NATS_DTYPE_BF16) {
    hipLaunchKernelGGL(roles_kernel<true>, grid, dim3(256), 0, st, logits, B, S, H_kv, global_bias, force_first_global,
                       force_last_global, roles, one_hot);
  } else {
    hipLaunchKernelGGL(roles_kernel<false>, grid, dim3(256), 0, st, logits, B, S, H_kv, global_bias,
                       force_first_global, force_last_global, roles, one_hot);
  }
  NATS_CHECK_LAUNCH("roles_kernel");
  return NATS_OK;
}

static int check_cw(const char* who, int64_t C, int64_t W) {
  NATS_REQUIRE(is_pow2(C), NATS_ERR_UNSUPPORTED, "%s: chunk size %lld is not a power of two", who, (long long)C);
  NATS_REQUIRE(W >= 0 && W % C == 0, NATS_ERR_BAD_SHAPE, "%s: window %lld is not a multiple of chunk size %lld", who,
               (long long)W, (long long)C);
  return NATS_OK;
}

extern "C" int nats_role_scan(const uint8_t* roles, int64_t B, int64_t H_kv, int64_t S, int64_t W, int64_t C,
                              int64_t* end_idx, int32_t* vis_lim, void* stream) {
  NATS_REQUIRE(roles, NATS_ERR_NULL_POINTER, "nats_role_scan: roles must not be NULL");
  NATS_REQUIRE(B > 0 && H_kv > 0 && S > 0 && S < (int64_t(1) << 30), NATS_ERR_BAD_SHAPE,
               "nats_role_scan: B=%lld H_kv=%lld S=%lld", (long long)B, (long long)H_kv, (long long)S);
  if (int rc = check_cw("nats_role_scan", C, W)) return rc;
  return launch_role_scan(roles, B * H_kv, S, W, C, end_idx, vis_lim, static_cast<hipStream_t>(stream));
}

extern "C" int nats_prefill_mask(const int32_t* vis_lim, int64_t B, int64_t H_kv, int64_t L, int64_t C, uint8_t* mask,
                                 void* stream) {
  NATS_REQUIRE(vis_lim && mask, NATS_ERR_NULL_POINTER, "nats_prefill_mask: NULL pointer");
  NATS_REQUIRE(B > 0 && H_kv > 0 && L > 0 && L <= 65535, NATS_ERR_BAD_SHAPE, "nats_prefill_mask: B=%lld H_kv=%lld L=%lld",
               (long long)B, (long long)H_kv, (long long)L);
  NATS_REQUIRE(is_pow2(C), NATS_ERR_UNSUPPORTED, "nats_prefill_mask: chunk size %lld", (long long)C);
  NATS_REQUIRE(B * H_kv <= 65535, NATS_ERR_BAD_SHAPE, "nats_prefill_mask: too many streams");
  int64_t S = (L + C - 1) / C;
  dim3 grid((unsigned)((L + 255) / 256), (unsigned)L, (unsigned)(B * H_kv));
  hipLaunchKernelGGL(mask_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), vis_lim, S, L, ilog2(C), mask);
  NATS_CHECK_LAUNCH("mask_kernel");
  return NATS_OK;
}

extern "C" int nats_prefill_tile_map(const int32_t* vis_lim, int64_t B, int64_t H_kv, int64_t L, int64_t C,
                                     void* tile_lim_ws, uint8_t* tiles, void* stream) {
  NATS_REQUIRE(vis_lim && tiles && tile_lim_ws, NATS_ERR_NULL_POINTER, "nats_prefill_tile_map: NULL pointer");
  NATS_REQUIRE(B > 0 && H_kv > 0 && L > 0, NATS_ERR_BAD_SHAPE, "nats_prefill_tile_map: B=%lld H_kv=%lld L=%lld",
               (long long)B, (long long)H_kv, (long long)L);
  NATS_REQUIRE(is_pow2(C), NATS_ERR_UNSUPPORTED, "nats_prefill_tile_map: chunk size %lld", (long long)C);
  int64_t S = (L + C - 1) / C;
  int64_t T = (L + kTile - 1) / kTile;
  NATS_REQUIRE(T <= 65535 && B * H_kv <= 65535, NATS_ERR_BAD_SHAPE, "nats_prefill_tile_map: grid too large");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (int rc = launch_tile_lim(vis_lim, B * H_kv, S, T, C, static_cast<int2*>(tile_lim_ws), st)) return rc;
  dim3 grid((unsigned)((T + 255) / 256), (unsigned)T, (unsigned)(B * H_kv));
  hipLaunchKernelGGL(tile_map_kernel, grid, dim3(256), 0, st, static_cast<const int2*>(tile_lim_ws), T, ilog2(C), tiles);
  NATS_CHECK_LAUNCH("tile_map_kernel");
  return NATS_OK;
}
