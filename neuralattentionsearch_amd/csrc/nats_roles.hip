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
// Reverse scan per (b, h) in blocks of 64 slots with a ballot per block.
// end_idx[n] = first global slot >= n, the last slot counting as global (components/masks/utils.py:85-87).
// vis_lim[n] = last query slot that sees key slot n:
//   global -> INT32_MAX, sliding window -> n + W / C, local -> end_idx[n]
// (components/masks/utils.py:92 and components/cache/nats_chunk_layer_cache.py:603-611).
// ---------------------------------------------------------------------------------------------------
// A workgroup takes kScanWaves * kScanSpan consecutive slots of one stream, a wavefront kScanSpan of them: it first
// looks for the first global slot of its span (and the last wavefront for the first one behind the workgroup's slots,
// which is usually a block or two away), then walks its span from the end with what follows it as the carry.
constexpr int kScanWaves = 16;
constexpr int kScanSpan = 256;

__global__ __launch_bounds__(kScanWaves * kWave) void role_scan_kernel(const uint8_t* __restrict__ roles, int64_t S,
                                                                       int32_t wc, int64_t* __restrict__ end_idx,
                                                                       int32_t* __restrict__ vis_lim,
                                                                       int32_t* __restrict__ first_global) {
  __shared__ int64_t first_g[kScanWaves + 1];
  const int64_t stream = blockIdx.x;
  const uint8_t* r = roles + stream * S;
  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int64_t seg0 = int64_t(blockIdx.y) * (kScanWaves * kScanSpan);
  const int64_t span0 = seg0 + wave * kScanSpan;
  const int64_t span1 = min(span0 + kScanSpan, S);
  auto first_global_in = [&](int64_t lo, int64_t hi) {  // first global slot in [lo, hi), or S
    for (int64_t b = lo; b < hi; b += kWave) {
      const int64_t n = b + lane;
      const bool is_g = n < hi && (r[n] == NATS_ROLE_GLOBAL || n == S - 1);
      const uint64_t bits = __ballot(is_g);
      if (bits) return b + __builtin_ctzll(bits);
    }
    return S;
  };
  const int64_t mine = first_global_in(span0, span1);
  if (lane == 0) first_g[wave] = mine;
  if (wave == kScanWaves - 1) {
    const int64_t behind = first_global_in(min(seg0 + kScanWaves * kScanSpan, S), S);
    if (lane == 0) first_g[kScanWaves] = behind < S ? behind : S - 1;
  }
  __syncthreads();
  int64_t carry = first_g[kScanWaves];
  for (int w = kScanWaves - 1; w > wave; --w)
    if (first_g[w] < S) carry = first_g[w];
  if (span0 < S) {
    for (int64_t base = span0 + ((span1 - 1 - span0) / kWave) * kWave; base >= span0; base -= kWave) {
      int64_t n = base + lane;
      bool in = n < span1;
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
  if (first_global && blockIdx.y == 0 && wave == 0 && lane == 0) first_global[stream] = int32_t(carry);  // end_idx[0]
}

// Per key row the last query token (counted from the start of the open-chunk region) that sees it, and
// per 64-row key tile the largest and the smallest of these limits: tile_lim[stream][t] = {max, min}.
// A query tile whose first token is r0 must load key tile t iff max >= r0; every score of the pair is
// unmasked iff all keys of t lie at or before the query tile's first token and min >= its last token.
//
// Rows of the region (row >= base) follow the roles of the segment: a slot visible up to query slot
// vis_lim is visible up to token (vis_lim + 1) * C - 1.  Rows below base are what an earlier segment left
// in the cache (components/cache/nats_chunk_layer_cache.py:462-511, 658-713):
//   ring rows [0, W)            valid and not older than the window for that query
//   rows [W, gmin)              valid_tokens as stored
//   rows [gmin, size_global)    always (kept globals)
//   rows [size_global, +local)  up to the first global slot of the segment
//   beyond                      never (rows that longer heads use)
template <bool kPast>
__global__ __launch_bounds__(256) void key_lim_kernel(KeyLimArgs a) {
  const int stream = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int tile = blockIdx.x * 4 + wave;
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x < kTicketQueues && a.ticket) a.ticket[threadIdx.x * kTicketStride] = 0;
  if (tile >= a.Tk) return;
  const int row = tile * kTile + lane;
  int32_t lim = -1;
  // Slot-level limit of this lane's row from the roles themselves (as role_scan_kernel computes it: global ->
  // INT32_MAX, sliding window -> slot + W / C, local -> the first global slot at or after it, the last slot counting
  // as global): the wavefront's rows span at most 64 consecutive slots, so one ballot over the 64 slots from its first
  // one answers most lanes, and the blocks that follow answer the rest with their first global slot.
  int32_t v_inline = 0;
  // (x / C for x >= 0; a shift when the chunk size is a power of two)
  auto slot_of = [&](int x) { return a.c_shift >= 0 ? x >> a.c_shift : x / a.C; };
  if (!kPast && a.roles) {
    const uint8_t* r = a.roles + (int64_t)stream * a.S;
    const bool in = row < a.N;
    const int slot = in ? slot_of(row) : 0;
    const int s0 = slot_of(tile * kTile);  // slot of lane 0 (the tile starts inside N)
    const uint8_t role = in ? r[slot] : uint8_t(NATS_ROLE_GLOBAL);
    const bool want = in && role == NATS_ROLE_LOCAL;
    int g = -1;
    if (__ballot(want)) {
      for (int blk = s0; blk < a.S; blk += kWave) {
        const int n = blk + lane;
        const bool is_g = n < a.S && (r[n] == NATS_ROLE_GLOBAL || n == a.S - 1);
        const uint64_t bits = __ballot(is_g);
        if (want && g < 0) {
          const int rel = slot - blk;  // 0 .. 63 in the first block, negative afterwards
          const uint64_t ahead = rel > 0 ? bits >> rel : bits;
          if (ahead) g = (rel > 0 ? slot : blk) + __builtin_ctzll(ahead);
        }
        if (!__ballot(want && g < 0)) break;
      }
    }
    v_inline = role == NATS_ROLE_GLOBAL ? kLimGlobal : role == NATS_ROLE_SW ? slot + slot_of(a.W) : g;
  }
  if (row < a.N) {
    if (!kPast || row >= a.base) {
      int32_t v = (!kPast && a.roles) ? v_inline : a.vis_lim[(int64_t)stream * a.S + slot_of(row - a.base)];
      int64_t t = (int64_t(v) + 1) * a.C - 1;
      lim = (v == kLimGlobal || t >= kLimGlobal) ? kLimGlobal : int32_t(t);
    } else {
      const int b = stream / a.Hkv, h = stream % a.Hkv;
      const bool val = a.valid[b * a.valid_s_b + h * a.valid_s_h + row] != 0;
      const int C = a.C;
      if (a.token_mode) {
        // The per-token cache (components/cache/nats_layer_cache.py:469-517, 603-649).  Its limits count the
        // queries of this call (i = r - old_fill), hence the + old_fill.
        if (row < a.W) {
          if (a.seen < a.W) {
            // ring not yet full: the columns of the tokens seen so far are overwritten with an age test, valid
            // or not (:612-619); the others keep valid_tokens
            lim = row < a.seen ? a.W - 1 - row + a.old_fill : (val ? kLimGlobal : -1);
          } else {
            // slot tail + 1 holds the oldest token, seen by the first query only (:621-647)
            lim = val ? (row + a.W - 1 - a.tail) % a.W + a.old_fill : -1;
          }
        } else if (row < a.gmin) {
          lim = val ? kLimGlobal : -1;
        } else {
          // rows [gmin, base): global rows always, local rows up to the first global token of the block,
          // nothing beyond a head's own rows (:502-516)
          const int64_t sg = a.size_global[stream], sl = a.size_local[stream];
          if (row >= sg + sl) {
            lim = -1;
          } else if (row >= sg) {
            lim = a.first_global[stream] + a.old_fill;
          } else {
            lim = kLimGlobal;
          }
        }
      } else if (row < a.W) {
        const int s = slot_of(row);
        if (!val) {
          lim = -1;
        } else if (a.seen >= a.W) {
          lim = ((s + 1) * C + a.W - 1 - a.tail) % a.W;  // queue offset of the slot's newest row (:687-707)
        } else if (s < a.seen / C) {
          int t = (a.W / C - s) * C - 1 - a.fill_last;  // (r + fill_last) / C + s < W / C  (:666-676)
          lim = t < 0 ? -1 : t;
        } else {
          lim = kLimGlobal;
        }
      } else {
        const int ncc = (a.base - a.gmin) / C;
        if (row < a.gmin || row >= a.gmin + ncc * C) {
          lim = val ? kLimGlobal : -1;
        } else {
          const int cc = (row - a.gmin) / C;
          const int64_t sg = a.size_global[stream], sl = a.size_local[stream];
          const int64_t lo = (sg - a.gmin) / C, hi = (sg + sl - a.gmin) / C;
          if (cc >= hi) {
            lim = -1;
          } else if (cc < lo) {
            lim = kLimGlobal;
          } else {
            lim = (a.first_global[stream] + 1) * C - 1;  // query slot <= first global slot of the segment (:480-494)
          }
        }
      }
    }
    a.tok_lim[(int64_t)stream * a.N + row] = lim;
  }
  int32_t mx = lim, mn = row < a.N ? lim : kLimGlobal;
#pragma unroll
  for (int off = kGranule / 2; off >= 1; off >>= 1) {
    mx = max(mx, __shfl_xor(mx, off));
    mn = min(mn, __shfl_xor(mn, off));
  }
  if ((lane & (kGranule - 1)) == 0)
    a.gran_lim[((int64_t)stream * a.Tk + tile) * (kTile / kGranule) + lane / kGranule] = make_int2(mx, mn);
#pragma unroll
  for (int off = 32; off >= kGranule; off >>= 1) {
    mx = max(mx, __shfl_xor(mx, off));
    mn = min(mn, __shfl_xor(mn, off));
  }
  if (lane == 0) a.tile_lim[(int64_t)stream * a.Tk + tile] = make_int2(mx, mn);
  if (a.tile_long) {
    const bool is_long = row < a.N && lim >= 0 && lim >= row - a.base + a.t_long;
    const bool kind_a = is_long && lim == kLimGlobal;
    const bool kind_b = is_long && !kind_a;
    int mb = kind_b ? lim : -1;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) mb = max(mb, __shfl_xor(mb, off));
    const int na = __builtin_popcountll(__ballot(kind_a)), nb = __builtin_popcountll(__ballot(kind_b));
    if (lane == 0) a.tile_long[(int64_t)stream * a.Tk + tile] = make_int4(na, nb, mb, 0);
  }
  if (stream == 0 && tile == 0 && lane == 0) a.tok_lim[(int64_t)gridDim.y * a.N] = -1;
}

// token-level mask from the per-row limits: query i of the segment is region token r = r_begin + i
__global__ void mask_rows_kernel(const int32_t* __restrict__ tok_lim, int64_t N, int64_t x_len, int64_t base,
                                 int64_t r_begin, uint8_t* __restrict__ mask) {
  int64_t row = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  int64_t i = blockIdx.y;
  int64_t stream = blockIdx.z;
  if (row >= N) return;
  int64_t r = r_begin + i;
  bool vis = r <= int64_t(tok_lim[stream * N + row]) && row - base <= r;
  mask[(stream * x_len + i) * N + row] = vis ? 1 : 0;
}

__global__ void tile_map_kernel(const int2* __restrict__ tile_lim, int64_t T, uint8_t* __restrict__ tiles) {
  int64_t kt = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  int64_t qt = blockIdx.y;
  int64_t stream = blockIdx.z;
  if (kt >= T) return;
  bool visit = kt <= qt && int64_t(tile_lim[stream * T + kt].x) >= qt * kTile;
  tiles[(stream * T + qt) * T + kt] = visit ? 1 : 0;
}

int launch_role_scan(const uint8_t* roles, int64_t n_streams, int64_t S, int64_t W, int64_t C, int64_t* end_idx,
                     int32_t* vis_lim, int32_t* first_global, hipStream_t st) {
  const int64_t n_seg = (S + kScanWaves * kScanSpan - 1) / (kScanWaves * kScanSpan);
  NATS_REQUIRE(n_seg <= 65535, NATS_ERR_BAD_SHAPE, "role_scan_kernel: %lld role slots per stream", (long long)S);
  hipLaunchKernelGGL(role_scan_kernel, dim3((unsigned)n_streams, (unsigned)n_seg), dim3(kScanWaves * kWave), 0, st, roles, S,
                     int32_t(W / C), end_idx, vis_lim, first_global);
  NATS_CHECK_LAUNCH("role_scan_kernel");
  return NATS_OK;
}

int launch_key_lim(const KeyLimArgs& a, int64_t n_streams, bool past, hipStream_t st) {
  NATS_REQUIRE(n_streams <= 65535, NATS_ERR_BAD_SHAPE, "too many (batch, kv head) streams: %lld", (long long)n_streams);
  dim3 grid((unsigned)((a.Tk + 3) / 4), (unsigned)n_streams);
  if (past) {
    hipLaunchKernelGGL(key_lim_kernel<true>, grid, dim3(256), 0, st, a);
  } else {
    hipLaunchKernelGGL(key_lim_kernel<false>, grid, dim3(256), 0, st, a);
  }
  NATS_CHECK_LAUNCH("key_lim_kernel");
  return NATS_OK;
}

PrefillWorkspace carve_prefill_workspace(void* ws, int64_t n_streams, int64_t S, int64_t N) {
  auto up = [](size_t x) { return (x + 255) & ~size_t(255); };
  const int64_t Tk = (N + kTile - 1) / kTile;
  PrefillWorkspace w;
  char* p = static_cast<char*>(ws);
  size_t off = 0;
  w.vis_lim = reinterpret_cast<int32_t*>(p + off);
  off += up((size_t)(n_streams * S) * sizeof(int32_t));
  w.first_global = reinterpret_cast<int32_t*>(p + off);
  off += up((size_t)n_streams * sizeof(int32_t));
  w.tok_lim = reinterpret_cast<int32_t*>(p + off);
  off += up((size_t)(n_streams * N + 1) * sizeof(int32_t));
  w.tile_lim = reinterpret_cast<int2*>(p + off);
  off += up((size_t)(n_streams * Tk) * sizeof(int2));
  w.gran_lim = reinterpret_cast<int2*>(p + off);
  off += up((size_t)(n_streams * Tk * (kTile / kGranule)) * sizeof(int2));
  w.ticket = reinterpret_cast<int32_t*>(p + off);
  off += up(8 * 32 * sizeof(int32_t));  // eight counters, 128 bytes apart
  w.long_cap = (Tk + 1) * kTile;
  w.n_gran = Tk * (kTile / kGranule);
  w.n_rtile = Tk + 2;
  w.long_rows = reinterpret_cast<int32_t*>(p + off);
  off += up((size_t)(n_streams * 2 * w.long_cap) * sizeof(int32_t));
  w.long_lim = reinterpret_cast<int32_t*>(p + off);
  off += up((size_t)(n_streams * 2 * w.long_cap) * sizeof(int32_t));
  w.tile_long = reinterpret_cast<int4*>(p + off);
  off += up((size_t)(n_streams * Tk) * sizeof(int4));
  w.long_before = reinterpret_cast<int32_t*>(p + off);
  off += up((size_t)(n_streams * 2 * (w.n_gran + 1)) * sizeof(int32_t));
  w.long_alive = reinterpret_cast<int32_t*>(p + off);
  off += up((size_t)(n_streams * w.n_rtile) * sizeof(int32_t));
  w.bytes = off;
  return w;
}

// ---------------------------------------------------------------------------------------------------
// Long-lived rows.  With chunks shorter than a 16-row granule most granules far behind a query hold a row or two
// that it still sees (a global token among sliding-window tokens), and walking them granule by granule loads and
// multiplies mostly invisible rows.  A row is long-lived when some query more than t_long tokens after it may see it:
// tok_lim[n] >= (n - base) + t_long.  A query group whose first token is r0 finds, among the rows below
// base + r0 - t_long, its visible rows among the long-lived ones only (any other row there has tok_lim < r0).
// Per stream the kernel writes two lists of row ids with their limits, each in ascending row order:
//   A  long-lived rows that every later query sees (global tokens, kept cache rows);
//   B  long-lived rows with a last query that sees them (local tokens far from their next global token, ring rows):
//      the entries before the first one at which the running maximum of the limits along the list reaches r0 are
//      invisible from r0 on, and `alive` holds that first entry for every 64-token region tile;
// and for each list the number of entries before every granule.  The attention kernel gathers the entries of A
// below its first granule-walked row, and those of B from `alive` on, 64 to a tile.
// A wavefront per 64-row tile; what lies before a tile comes from the per-tile counts the key-limit kernel left.
// ---------------------------------------------------------------------------------------------------
constexpr int kLongWaves = 16;  // 64-row tiles per workgroup

__global__ __launch_bounds__(kLongWaves * kWave) void long_rows_kernel(const int32_t* __restrict__ tok_lim,
                                                                       const int4* __restrict__ tile_long, int N, int Tk,
                                                                       int base, int t_long, int n_gran, int long_cap,
                                                                       int n_rtile, int32_t* __restrict__ long_rows,
                                                                       int32_t* __restrict__ long_lim,
                                                                       int32_t* __restrict__ long_before,
                                                                       int32_t* __restrict__ long_alive) {
  __shared__ int red_a[kLongWaves], red_b[kLongWaves], red_m[kLongWaves];
  const int ks = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int t0 = blockIdx.x * kLongWaves;  // first tile of this workgroup
  const int tile = t0 + wave;
  const int4* tl = tile_long + (int64_t)ks * Tk;
  // entries of both lists, and the greatest limit in B, in the tiles before this workgroup's
  int sa = 0, sb = 0, sm = -1;
  for (int t = tid; t < t0; t += kLongWaves * kWave) {
    const int4 c = tl[t];
    sa += c.x;
    sb += c.y;
    sm = max(sm, c.z);
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    sa += __shfl_xor(sa, o);
    sb += __shfl_xor(sb, o);
    sm = max(sm, __shfl_xor(sm, o));
  }
  if (lane == 0) {
    red_a[wave] = sa;
    red_b[wave] = sb;
    red_m[wave] = sm;
  }
  __syncthreads();
  int base_a = 0, base_b = 0, run_max = -1;
#pragma unroll
  for (int w = 0; w < kLongWaves; ++w) {
    base_a += red_a[w];
    base_b += red_b[w];
    run_max = max(run_max, red_m[w]);
  }
  // ... and in the tiles of this workgroup before this wavefront's
  {
    int4 c = make_int4(0, 0, -1, 0);
    if (lane < wave && t0 + lane < Tk) c = tl[t0 + lane];
    int ca = c.x, cb = c.y, cm = c.z;
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) {
      ca += __shfl_xor(ca, o);
      cb += __shfl_xor(cb, o);
      cm = max(cm, __shfl_xor(cm, o));
    }
    base_a += __shfl(ca, 0);
    base_b += __shfl(cb, 0);
    run_max = max(run_max, __shfl(cm, 0));
  }
  int32_t* rows_a = long_rows + (int64_t)ks * 2 * long_cap;
  int32_t* lims_a = long_lim + (int64_t)ks * 2 * long_cap;
  int32_t* rows_b = rows_a + long_cap;
  int32_t* lims_b = lims_a + long_cap;
  int32_t* before_a = long_before + (int64_t)ks * 2 * (n_gran + 1);
  int32_t* before_b = before_a + (n_gran + 1);
  int32_t* alive = long_alive + (int64_t)ks * n_rtile;
  if (tile < Tk) {
    const int row = tile * kTile + lane;
    const int lim = row < N ? tok_lim[(int64_t)ks * N + row] : -1;
    const bool is_long = lim >= 0 && lim >= row - base + t_long;
    const bool kind_a = is_long && lim == kLimGlobal;
    const bool kind_b = is_long && !kind_a;
    const uint64_t bits_a = __ballot(kind_a), bits_b = __ballot(kind_b);
    const uint64_t below = (uint64_t(1) << lane) - 1;
    const int off_a = base_a + __builtin_popcountll(bits_a & below);
    const int off_b = base_b + __builtin_popcountll(bits_b & below);
    if ((lane & (kGranule - 1)) == 0) {
      before_a[row / kGranule] = off_a;
      before_b[row / kGranule] = off_b;
    }
    if (kind_a) {
      rows_a[off_a] = row;
      lims_a[off_a] = lim;
    }
    // running maximum of the limits of B up to and without this lane's row
    int incl = kind_b ? lim : -1;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const int y = __shfl_up(incl, o);
      if (lane >= o) incl = max(incl, y);
    }
    int prev = __shfl_up(incl, 1);
    if (lane == 0) prev = -1;
    prev = max(prev, run_max);
    if (kind_b) {
      rows_b[off_b] = row;
      lims_b[off_b] = lim;
      // this entry is the first that matters to the region tiles whose first token lies in (prev, max(prev, lim)]
      const int t_lo = prev < 0 ? 0 : prev / kTile + 1;
      const int t_hi = min(max(prev, lim) / kTile, n_rtile - 1);
      for (int t = t_lo; t <= t_hi; ++t) alive[t] = off_b;
    }
    if (tile == Tk - 1) {
      // the ends of the lists: totals, padding (A is read in whole tiles, a tile of B may start at any entry), and
      // the region tiles that begin behind every limit in B
      const int n_a = base_a + __builtin_popcountll(bits_a), n_b = base_b + __builtin_popcountll(bits_b);
      const int all_max = max(run_max, __shfl(incl, kWave - 1));
      if (lane == 0) {
        before_a[n_gran] = n_a;
        before_b[n_gran] = n_b;
      }
      for (int i = n_a + lane; i < (n_a + kTile - 1) / kTile * kTile; i += kWave) {
        rows_a[i] = 0x7fffffff;
        lims_a[i] = -1;
      }
      rows_b[n_b + lane] = 0x7fffffff;
      lims_b[n_b + lane] = -1;
      for (int t = (all_max < 0 ? 0 : all_max / kTile + 1) + lane; t < n_rtile; t += kWave) alive[t] = n_b;
    }
  }
}

int launch_long_rows(const PrefillWorkspace& w, int64_t n_streams, int64_t N, int64_t base, int64_t W, hipStream_t st) {
  NATS_REQUIRE(n_streams <= 65535, NATS_ERR_BAD_SHAPE, "long_rows_kernel: %lld streams", (long long)n_streams);
  const int64_t Tk = (N + kTile - 1) / kTile;
  dim3 grid((unsigned)((Tk + kLongWaves - 1) / kLongWaves), (unsigned)n_streams);
  // (the threshold is the one the key-limit kernel counted the tiles' rows with)
  hipLaunchKernelGGL(long_rows_kernel, grid, dim3(kLongWaves * kWave), 0, st, w.tok_lim, w.tile_long, (int)N, (int)Tk,
                     (int)base, (int)long_row_threshold(W), (int)w.n_gran, (int)w.long_cap, (int)w.n_rtile, w.long_rows, w.long_lim,
                     w.long_before, w.long_alive);
  NATS_CHECK_LAUNCH("long_rows_kernel");
  return NATS_OK;
}

// roles -> vis_lim, first_global -> tok_lim, tile_lim.  `past` may be NULL (prefill from an empty cache).
int prepare_key_limits(const uint8_t* roles, int64_t B, int64_t H_kv, int64_t S, int64_t N, int64_t C, int64_t W,
                       const PastView* past, const PrefillWorkspace& w, hipStream_t st) {
  const int64_t n_streams = B * H_kv;
  KeyLimArgs a{};
  // A prefill from an empty cache needs the scan's result only inside the key-limit kernel, which then searches the
  // roles itself (one launch less); streams so long that a run of local slots could make that search slow, and
  // segments over a filled cache (which also need the first global slot), take the scan kernel.
  const bool inline_scan = past == nullptr && S <= 8192;
  if (inline_scan) {
    a.roles = roles;
  } else if (int rc = launch_role_scan(roles, n_streams, S, W, C, nullptr, w.vis_lim, w.first_global, st)) {
    return rc;
  }
  a.vis_lim = w.vis_lim;
  a.first_global = w.first_global;
  a.tok_lim = w.tok_lim;
  a.tile_lim = w.tile_lim;
  a.gran_lim = w.gran_lim;
  a.ticket = w.ticket;
  a.tile_long = w.tile_long;
  a.t_long = (int)long_row_threshold(W);
  a.Hkv = (int)H_kv; a.S = (int)S; a.N = (int)N; a.Tk = (int)((N + kTile - 1) / kTile);
  a.c_shift = is_pow2(C) ? ilog2(C) : -1; a.C = (int)C; a.W = (int)W;
  if (past) {
    a.valid = past->valid; a.valid_s_b = past->valid_s_b; a.valid_s_h = past->valid_s_h;
    a.size_global = past->size_global; a.size_local = past->size_local;
    a.base = (int)past->base; a.gmin = (int)past->gmin; a.tail = (int)past->tail; a.seen = (int)past->seen;
    a.fill_last = (int)past->fill_last;
    a.old_fill = (int)past->old_fill; a.token_mode = past->token_mode;
  }
  return launch_key_lim(a, n_streams, past != nullptr, st);
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
  NATS_REQUIRE(C > 0 && C < (int64_t(1) << 30), NATS_ERR_BAD_SHAPE, "%s: chunk size %lld", who, (long long)C);
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
  return launch_role_scan(roles, B * H_kv, S, W, C, end_idx, vis_lim, nullptr, static_cast<hipStream_t>(stream));
}

static int launch_mask_rows(const PrefillWorkspace& w, int64_t n_streams, int64_t N, int64_t x_len, int64_t base,
                            int64_t r_begin, uint8_t* mask, hipStream_t st) {
  NATS_REQUIRE(x_len <= 65535 && n_streams <= 65535, NATS_ERR_BAD_SHAPE, "mask output: grid too large");
  dim3 grid((unsigned)((N + 255) / 256), (unsigned)x_len, (unsigned)n_streams);
  hipLaunchKernelGGL(mask_rows_kernel, grid, dim3(256), 0, st, w.tok_lim, N, x_len, base, r_begin, mask);
  NATS_CHECK_LAUNCH("mask_rows_kernel");
  return NATS_OK;
}

extern "C" int nats_prefill_mask(const uint8_t* roles, int64_t B, int64_t H_kv, int64_t L, int64_t C, int64_t W,
                                 uint8_t* mask, void* workspace, size_t workspace_bytes, void* stream) {
  NATS_REQUIRE(roles && mask && workspace, NATS_ERR_NULL_POINTER, "nats_prefill_mask: NULL pointer");
  NATS_REQUIRE(B > 0 && H_kv > 0 && L > 0, NATS_ERR_BAD_SHAPE, "nats_prefill_mask: B=%lld H_kv=%lld L=%lld",
               (long long)B, (long long)H_kv, (long long)L);
  if (int rc = check_cw("nats_prefill_mask", C, W)) return rc;
  const int64_t S = (L + C - 1) / C;
  PrefillWorkspace w = carve_prefill_workspace(workspace, B * H_kv, S, L);
  NATS_REQUIRE(workspace_bytes >= w.bytes, NATS_ERR_WORKSPACE, "nats_prefill_mask: workspace %zu bytes < %zu",
               workspace_bytes, w.bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (int rc = prepare_key_limits(roles, B, H_kv, S, L, C, W, nullptr, w, st)) return rc;
  return launch_mask_rows(w, B * H_kv, L, L, 0, 0, mask, st);
}

extern "C" int nats_prefill_tile_map(const uint8_t* roles, int64_t B, int64_t H_kv, int64_t L, int64_t C, int64_t W,
                                     uint8_t* tiles, void* workspace, size_t workspace_bytes, void* stream) {
  NATS_REQUIRE(roles && tiles && workspace, NATS_ERR_NULL_POINTER, "nats_prefill_tile_map: NULL pointer");
  NATS_REQUIRE(B > 0 && H_kv > 0 && L > 0, NATS_ERR_BAD_SHAPE, "nats_prefill_tile_map: B=%lld H_kv=%lld L=%lld",
               (long long)B, (long long)H_kv, (long long)L);
  if (int rc = check_cw("nats_prefill_tile_map", C, W)) return rc;
  const int64_t S = (L + C - 1) / C;
  const int64_t T = (L + kTile - 1) / kTile;
  NATS_REQUIRE(T <= 65535 && B * H_kv <= 65535, NATS_ERR_BAD_SHAPE, "nats_prefill_tile_map: grid too large");
  PrefillWorkspace w = carve_prefill_workspace(workspace, B * H_kv, S, L);
  NATS_REQUIRE(workspace_bytes >= w.bytes, NATS_ERR_WORKSPACE, "nats_prefill_tile_map: workspace %zu bytes < %zu",
               workspace_bytes, w.bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (int rc = prepare_key_limits(roles, B, H_kv, S, L, C, W, nullptr, w, st)) return rc;
  dim3 grid((unsigned)((T + 255) / 256), (unsigned)T, (unsigned)(B * H_kv));
  hipLaunchKernelGGL(tile_map_kernel, grid, dim3(256), 0, st, w.tile_lim, T, tiles);
  NATS_CHECK_LAUNCH("tile_map_kernel");
  return NATS_OK;
}

int nats::check_past_state(const char* who, const nats_past_state* ps, int64_t x_len, int64_t C, int64_t W) {
  NATS_REQUIRE(ps, NATS_ERR_NULL_POINTER, "%s: NULL past state", who);
  NATS_REQUIRE(x_len > 0, NATS_ERR_BAD_SHAPE, "%s: x_len=%lld", who, (long long)x_len);
  NATS_REQUIRE(ps->update_chunk >= 0 && (ps->update_chunk == 0 || (C == 1 && ps->update_chunk <= W)), NATS_ERR_BAD_SHAPE,
               "%s: update_chunk=%lld needs chunk size 1 and a window of at least that many tokens", who,
               (long long)ps->update_chunk);
  const int64_t fill_cap = ps->update_chunk ? ps->update_chunk : C;  // pending tokens stay below one (update) chunk
  NATS_REQUIRE(ps->old_fill >= 0 && ps->old_fill < fill_cap, NATS_ERR_BAD_SHAPE, "%s: old_fill=%lld outside [0, %lld)", who,
               (long long)ps->old_fill, (long long)fill_cap);
  NATS_REQUIRE(ps->n_ctx_data >= W + ps->old_fill && ps->n_ctx_data + x_len < (int64_t(1) << 30), NATS_ERR_BAD_SHAPE,
               "%s: n_ctx_data=%lld with window %lld and %lld open-chunk tokens", who, (long long)ps->n_ctx_data,
               (long long)W, (long long)ps->old_fill);
  NATS_REQUIRE(ps->gmin >= W && ps->gmin <= ps->n_ctx_data - ps->old_fill, NATS_ERR_BAD_SHAPE,
               "%s: gmin=%lld outside [W, first open-chunk row]", who, (long long)ps->gmin);
  NATS_REQUIRE(ps->tail >= 0 && (W == 0 ? ps->tail == 0 : ps->tail < W), NATS_ERR_BAD_SHAPE, "%s: tail=%lld", who,
               (long long)ps->tail);
  NATS_REQUIRE(ps->seen >= 0 && ps->fill_last >= 0 && ps->fill_last < fill_cap, NATS_ERR_BAD_SHAPE, "%s: seen=%lld fill_last=%lld",
               who, (long long)ps->seen, (long long)ps->fill_last);
  return NATS_OK;
}

extern "C" int nats_prefill_past_mask(const uint8_t* valid, const int64_t* size_global, const int64_t* size_local,
                                      const uint8_t* roles, int64_t B, int64_t H_kv, int64_t x_len, int64_t C, int64_t W,
                                      const nats_past_state* ps, const int64_t* valid_strides, uint8_t* mask,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  NATS_REQUIRE(valid && size_global && size_local && roles && mask && workspace && valid_strides, NATS_ERR_NULL_POINTER,
               "nats_prefill_past_mask: NULL pointer");
  NATS_REQUIRE(B > 0 && H_kv > 0, NATS_ERR_BAD_SHAPE, "nats_prefill_past_mask: B=%lld H_kv=%lld", (long long)B,
               (long long)H_kv);
  if (int rc = check_cw("nats_prefill_past_mask", C, W)) return rc;
  if (int rc = check_past_state("nats_prefill_past_mask", ps, x_len, C, W)) return rc;
  const int64_t fill = ps->old_fill + x_len;
  const int64_t S = (fill + C - 1) / C;
  const int64_t N = ps->n_ctx_data + x_len;
  PrefillWorkspace w = carve_prefill_workspace(workspace, B * H_kv, S, N);
  NATS_REQUIRE(workspace_bytes >= w.bytes, NATS_ERR_WORKSPACE, "nats_prefill_past_mask: workspace %zu bytes < %zu",
               workspace_bytes, w.bytes);
  PastView pv{valid, valid_strides[0], valid_strides[1], size_global, size_local, ps->n_ctx_data - ps->old_fill,
              ps->gmin, ps->tail, ps->seen, ps->fill_last, ps->old_fill, ps->update_chunk != 0};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (int rc = prepare_key_limits(roles, B, H_kv, S, N, C, W, &pv, w, st)) return rc;
  return launch_mask_rows(w, B * H_kv, N, x_len, pv.base, ps->old_fill, mask, st);
}
