// Shared helpers of the gfx950 NAtS kernels: error reporting, argument checks, small device utilities.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "nats_hip.h"

namespace nats {

// thread-local text behind nats_last_error()
char* error_buffer();
int fail(int code, const char* fmt, ...);

#define NATS_REQUIRE(cond, code, ...)           \
  do {                                          \
    if (!(cond)) return ::nats::fail((code), __VA_ARGS__); \
  } while (0)

#define NATS_CHECK_LAUNCH(what)                                                              \
  do {                                                                                       \
    hipError_t e__ = hipGetLastError();                                                      \
    if (e__ != hipSuccess) return ::nats::fail(NATS_ERR_LAUNCH, "%s: %s", (what), hipGetErrorString(e__)); \
  } while (0)

inline bool is_pow2(int64_t x) { return x > 0 && (x & (x - 1)) == 0; }
inline int ilog2(int64_t x) {
  int r = 0;
  while ((int64_t(1) << r) < x) ++r;
  return r;
}

constexpr int kWave = 64;
constexpr int kTile = 64;  // prefill tile edge (queries and keys)
constexpr int kGranule = 16;  // key rows whose limits are also summarised on their own (a quarter tile)
constexpr int32_t kLimGlobal = 0x7fffffff;
constexpr int kTicketQueues = 8;   // work counters of a prefill launch: one per XCD
constexpr int kTicketStride = 32;  // int32 entries between two of them (128 bytes: a memory line each)

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // 16 bytes as the native vector the streaming load / store builtins take

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// bf16 <-> f32 with round-to-nearest-even, bit exact with torch's conversion for finite values
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(uint32_t(b) << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return uint16_t((u >> 16) | 0x40u);  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return uint16_t(u >> 16);
}

// ---- key visibility limits shared by the prefill kernels and the mask / tile-map outputs ----------------
// State an earlier segment left in the cache, as the segment kernels need it.
struct PastView {
  const uint8_t* valid;  // valid_tokens, [B, H_kv, >= base]
  int64_t valid_s_b, valid_s_h;
  const int64_t* size_global;  // [B * H_kv]
  const int64_t* size_local;   // [B * H_kv]
  int64_t base;                // first cache row of the open-chunk region = n_ctx_data - old_fill
  int64_t gmin, tail, seen, fill_last;
  int64_t old_fill;   // region tokens cached before the segment
  int token_mode;     // the per-token cache (one role per token, `tail` = ring slot written last)
};

struct KeyLimArgs {
  const uint8_t* roles;         // [streams, S]; if set, the kernel derives the slot-level limits itself (no past only)
  const int32_t* vis_lim;       // [streams, S] slot-level limits of the segment's roles (used when roles is NULL)
  const int32_t* first_global;  // [streams] first global slot of the segment
  const uint8_t* valid;
  int64_t valid_s_b, valid_s_h;
  const int64_t* size_global;
  const int64_t* size_local;
  int32_t* tok_lim;  // [streams, N] out, followed by one entry that holds -1 (the limit of a row nobody sees)
  int2* tile_lim;    // [streams, Tk] out {max, min}
  int2* gran_lim;    // [streams, Tk * 4] out {max, min} of every 16 rows
  int32_t* ticket;   // out: one counter, set to zero (may be NULL)
  int4* tile_long;   // [streams, Tk] out (may be NULL): per 64-row tile the long-lived rows every later query sees, those
                     // with a last query, and the greatest limit among the latter (see long_rows_kernel)
  int t_long;
  int Hkv, S, N, Tk, c_shift, C, W;
  int base, gmin, tail, seen, fill_last;
  int old_fill, token_mode;
};

struct PrefillWorkspace {
  int32_t* vis_lim;
  int32_t* first_global;
  int32_t* tok_lim;
  int2* tile_lim;
  int2* gran_lim;
  int32_t* ticket;  // one counter, set to zero by the key-limit kernel (the attention kernel deals work from it)
  // long-lived rows (see long_rows_kernel): per stream two ascending lists of row ids with their limits (A: rows every
  // later query sees, B: rows with a last query), the number of entries
  // of each list before every 16-row granule, and for every 64-token region tile the first entry of B that matters
  int32_t* long_rows;    // [streams, 2, long_cap]
  int32_t* long_lim;     // [streams, 2, long_cap]
  int4* tile_long;       // [streams, Tk] counts of both kinds per 64-row tile, from the key-limit kernel
  int32_t* long_before;  // [streams, 2, n_gran + 1]
  int32_t* long_alive;   // [streams, n_rtile]
  int64_t long_cap;      // entries per list: N rounded up to whole tiles, plus one tile of padding
  int64_t n_gran;        // 16-row granules per stream
  int64_t n_rtile;       // entries of long_alive per stream
  size_t bytes;
};

PrefillWorkspace carve_prefill_workspace(void* ws, int64_t n_streams, int64_t S, int64_t N);
int prepare_key_limits(const uint8_t* roles, int64_t B, int64_t H_kv, int64_t S, int64_t N, int64_t C, int64_t W,
                       const PastView* past, const PrefillWorkspace& w, hipStream_t st);
int check_past_state(const char* who, const nats_past_state* ps, int64_t x_len, int64_t C, int64_t W);
// Fills the long-lived-row lists of the workspace from its key limits (after prepare_key_limits on the same stream).
int launch_long_rows(const PrefillWorkspace& w, int64_t n_streams, int64_t N, int64_t base, int64_t W, hipStream_t st);
// rows that a query more than this many tokens behind them may still see are long-lived
inline int64_t long_row_threshold(int64_t W) { return W + kGranule; }

// Orders LDS traffic between the lanes of one wavefront (no workgroup barrier needed for wave-private LDS).
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

}  // namespace nats
