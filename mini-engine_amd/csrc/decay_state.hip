// Linear attention with a fixed decay per head and a matrix of state per request and head (no softmax, no
// denominator):
//
//   S_t = decay_h * S_(t-1) + k_t v_t^T        (S: [d, dv], float32, kept in a slot between steps)
//   o_t = S_t^T q_t
//
// Three kernels a step (five where long prompts are walked a chunk at a time). `decay_state_prepare` turns the projections [T, H*d | H*d | H*dv | ...] into float32 q, k
// and v: an optional activation, an optional rotation of the first rd elements of q and k by the position's angles
// (either pairing), and a scale on k. `decay_state_scan` walks the new tokens of every item in order, from the state
// in the item's slot, and leaves the new state there. `decay_state_finish` norms the outputs (every head by its own
// root mean square, or all heads together with a weight), multiplies by the activation of the gate's projection and
// rounds to the compute type.
//
// Everything from the prepared q, k, v to the normed output is float32, and the scan adds in an order that depends on
// nothing but the head's sizes: a state column is owned by four lanes of one wave, each walking a quarter of the rows
// token by token, so a request's outputs are the same bits however its tokens are cut into steps and whatever else the
// step holds.
//
// The decay is carried as two floats (the nearest float and what it misses of the configured value), so that a state
// that has decayed over thousands of tokens has not drifted by the float's rounding of the decay times its age.
#include "common.h"

#define DS_MAX_D 256

enum DsAct { DS_ACT_NONE = 0, DS_ACT_SILU = 1, DS_ACT_SIGMOID = 2 };

__device__ __forceinline__ float ds_act(float z, int code) {
  if (code == DS_ACT_SILU) return z / (1.f + expf(-z));
  if (code == DS_ACT_SIGMOID) return 1.f / (1.f + expf(-z));
  return z;
}

// ---------------------------------------------------------------------------------------------- prepare
// One wave per (token, head) and kind (q, k, v). Output rows are padded: q32, k32 [T, H, dp] (zeros beyond d),
// v32 [T, H, dv].
template <typename T>
__global__ __launch_bounds__(256) void decay_state_prepare_kernel(
    const T* __restrict__ proj, int proj_cols, const float* __restrict__ rope_table, int rd, int pairing,
    const int* __restrict__ positions, float* __restrict__ q32, float* __restrict__ k32, float* __restrict__ v32,
    int num_tokens, int heads, int d, int dp, int dv, int act, float key_scale) {
  __shared__ float stage[4][DS_MAX_D];
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1);
  const long long unit = (long long)blockIdx.x * 4 + wave;
  if (unit >= (long long)num_tokens * heads * 3) return;
  const int kind = (int)(unit % 3), head = (int)((unit / 3) % heads), t = (int)(unit / 3 / heads);
  const int n = kind == 2 ? dv : d;
  const T* src = proj + (size_t)t * proj_cols + (kind == 0 ? (size_t)head * d
                                                 : kind == 1 ? (size_t)heads * d + (size_t)head * d
                                                             : (size_t)2 * heads * d + (size_t)head * dv);
  float* st = stage[wave];
  for (int i = lane; i < n; i += ME_WAVE) st[i] = ds_act(to_float(src[i]), act);
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): LDS writes of this wave are visible
  if (kind == 2) {
    float* dst = v32 + ((size_t)t * heads + head) * dv;
    for (int i = lane; i < dv; i += ME_WAVE) dst[i] = st[i];
    return;
  }
  float* dst = (kind == 0 ? q32 : k32) + ((size_t)t * heads + head) * dp;
  const float mult = kind == 1 ? key_scale : 1.f;
  const float* cs = rope_table ? rope_table + (size_t)positions[t] * rd : nullptr;  // [2, rd / 2] of this position
  const int half = rd / 2;
  for (int i = lane; i < dp; i += ME_WAVE) {
    float r = 0.f;
    if (i < d) {
      r = st[i];
      if (cs && i < rd) {
        const bool first = pairing == 0 ? i < half : (i & 1) == 0;
        const int j = pairing == 0 ? (first ? i : i - half) : i >> 1;
        const int other = pairing == 0 ? (first ? i + half : i - half) : i ^ 1;
        const float c = cs[j], sn = cs[half + j];
        r = first ? st[i] * c - st[other] * sn : st[i] * c + st[other] * sn;
      }
      r *= mult;
    }
    dst[i] = r;
  }
}

// ------------------------------------------------------------------------------------------------- scan
// A wave owns 16 * CPL columns of the state: lane = rg * 16 + c, rg = 0..3 the quarter of the rows (RPL rows a lane,
// 4 * RPL >= d; q32 and k32 rows are padded to 4 * RPL with zeros), c the lane's CPL neighbouring columns. The 16 lanes
// of a quarter read the same rows of k (and q): fetched from memory by every lane for itself, those reads kept the load
// path busy for longer than the arithmetic takes, so the chunked forms stage a chunk's rows in LDS once per block
// (a 2,048-token prompt, 16 heads of 128 x 128: the outputs 171 -> 114 us a layer), and the sums' form, which holds no
// q, gives a lane two columns (96 -> 57 us; the outputs' form with two columns a lane was slower, 193 us without the
// staging). A sum's order does not depend on any of this. The next token's q, k and v are requested before the current
// token's arithmetic. Three forms:
//
//   DS_WHOLE   grid (item, head, 64 columns): the item's new tokens in order, from the state in its slot, which is left
//              updated. The decay is applied as two floats. Decode steps and short portions.
//   DS_SUMS    grid (chunk of 64 tokens, head, 64 columns): the chunk's own sum  U = sum_s decay^(last - s) k_s v_s^T,
//              from nothing, into the chunk's place of `chunks` [chunk, head, d, dv]; no outputs.
//   DS_OUTPUTS the same grid: the chunk's tokens in order from the state at the chunk's start, which
//              `decay_state_chunk_starts_kernel` has put in the chunk's place; outputs, no state written.
//
// With the last two a long prompt is walked by all its chunks at once: sums, then the states at the chunks' starts (a
// pass over the chunks per element, with decay^64 worked out in double), then outputs. Inside a chunk the decay is one
// float: over 64 tokens what the float misses of the configured value stays below 1e-5 of a term.
#define DS_CHUNK 64
enum DsMode { DS_WHOLE = 0, DS_SUMS = 1, DS_OUTPUTS = 2 };

// The item and the tokens of chunk `c` (counted over all items of the step, ceil(tokens / 64) chunks an item).
__device__ __forceinline__ bool ds_chunk_tokens(const int* __restrict__ item_start, int items, int c, int& item, int& t0, int& t1) {
  int base = 0;
  for (int i = 0; i < items; ++i) {
    const int a = item_start[i], n = item_start[i + 1] - a;
    const int nc = (n + DS_CHUNK - 1) / DS_CHUNK;
    if (c < base + nc) {
      item = i;
      t0 = a + (c - base) * DS_CHUNK;
      t1 = min(t0 + DS_CHUNK, a + n);
      return true;
    }
    base += nc;
  }
  return false;
}

template <int RPL, int MODE, int CPL>
__global__ __launch_bounds__(256) void decay_state_scan_kernel(
    const float* __restrict__ q32, const float* __restrict__ k32, const float* __restrict__ v32, float* __restrict__ o32,
    float* __restrict__ state, float* __restrict__ chunks, const float* __restrict__ decay, const int* __restrict__ item_start,
    const int* __restrict__ state_slots, int items, int heads, int d, int dv) {
  constexpr int DP = 4 * RPL;
  constexpr int QUARTER = RPL + 4, LROW = 4 * QUARTER;  // a row of k or q in LDS: its four quarters 16 bytes apart from a
                                                        // multiple of 128, so that the four addresses of a read hit other banks
  extern __shared__ __attribute__((aligned(16))) float ds_lds[];  // the chunked forms: [64][LROW] of k, then of q
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1);
  const int head = blockIdx.y;
  const int col = ((blockIdx.z * 4 + wave) * 16 + (lane & 15)) * CPL, rg = lane >> 4;  // the first of this lane's columns
  const bool idle = (blockIdx.z * 4 + wave) * 16 * CPL >= dv;  // a wave beyond the last column
  if (MODE == DS_WHOLE && idle) return;
  bool has_col[CPL];
#pragma unroll
  for (int c = 0; c < CPL; ++c) has_col[c] = col + c < dv;
  int item = blockIdx.x, t0, t1;
  if (MODE == DS_WHOLE) {
    t0 = item_start[item], t1 = item_start[item + 1];
  } else if (!ds_chunk_tokens(item_start, items, blockIdx.x, item, t0, t1)) {
    return;
  }
  const int slot = state_slots[item];
  if (slot < 0 || t1 <= t0) return;  // (the same for every thread of the block)
  if (MODE != DS_WHOLE) {
    // The chunk's rows of k (and q) go to LDS once for the block's four waves: fetched by every lane for itself they
    // keep the load path busy for longer than the arithmetic takes (the 16 lanes of a quarter read the same 16 bytes).
    const int pieces = (t1 - t0) * (DP / 4);
    for (int idx = threadIdx.x; idx < pieces; idx += blockDim.x) {
      const int tt = idx / (DP / 4), p = idx % (DP / 4);
      const size_t row = ((size_t)(t0 + tt) * heads + head) * DP;
      const int at = tt * LROW + (p / (RPL / 4)) * QUARTER + (p % (RPL / 4)) * 4;
      *reinterpret_cast<float4*>(ds_lds + at) = reinterpret_cast<const float4*>(k32 + row)[p];
      if (MODE == DS_OUTPUTS) *reinterpret_cast<float4*>(ds_lds + DS_CHUNK * LROW + at) = reinterpret_cast<const float4*>(q32 + row)[p];
    }
    __syncthreads();
    if (idle) return;
  }
  const float lam = decay[head], lam_lo = MODE == DS_WHOLE ? decay[heads + head] : 0.f;
  float* srow = MODE == DS_WHOLE ? state + (((size_t)slot * heads + head) * d) * dv
                                 : chunks + (((size_t)blockIdx.x * heads + head) * d) * dv;  // [d, dv]
  float S[CPL][RPL];
#pragma unroll
  for (int c = 0; c < CPL; ++c)
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int i = rg * RPL + r;
      S[c][r] = MODE != DS_SUMS && has_col[c] && i < d ? srow[(size_t)i * dv + col + c] : 0.f;
    }
  float4 qn[RPL / 4], kn[RPL / 4];
  float vn[CPL];
  auto fetch = [&](int t) {
    const float4* kp = MODE == DS_WHOLE ? reinterpret_cast<const float4*>(k32 + ((size_t)t * heads + head) * DP + rg * RPL)
                                        : reinterpret_cast<const float4*>(ds_lds + (t - t0) * LROW + rg * QUARTER);
#pragma unroll
    for (int r = 0; r < RPL / 4; ++r) kn[r] = kp[r];
    if (MODE != DS_SUMS) {
      const float4* qp = MODE == DS_WHOLE ? reinterpret_cast<const float4*>(q32 + ((size_t)t * heads + head) * DP + rg * RPL)
                                          : reinterpret_cast<const float4*>(ds_lds + DS_CHUNK * LROW + (t - t0) * LROW + rg * QUARTER);
#pragma unroll
      for (int r = 0; r < RPL / 4; ++r) qn[r] = qp[r];
    }
#pragma unroll
    for (int c = 0; c < CPL; ++c) vn[c] = has_col[c] ? v32[((size_t)t * heads + head) * dv + col + c] : 0.f;
  };
  fetch(t0);
  for (int t = t0; t < t1; ++t) {
    float4 qc[RPL / 4], kc[RPL / 4];
#pragma unroll
    for (int r = 0; r < RPL / 4; ++r) kc[r] = kn[r];
    if (MODE != DS_SUMS) {
#pragma unroll
      for (int r = 0; r < RPL / 4; ++r) qc[r] = qn[r];
    }
    float vc[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) vc[c] = vn[c];
    if (t + 1 < t1) fetch(t + 1);
    float o[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) o[c] = 0.f;
#pragma unroll
    for (int r = 0; r < RPL / 4; ++r) {
      const float kk[4] = {kc[r].x, kc[r].y, kc[r].z, kc[r].w};
#pragma unroll
      for (int c = 0; c < CPL; ++c)
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const float s = S[c][4 * r + u];
          float sn = fmaf(lam, s, kk[u] * vc[c]);
          if (MODE == DS_WHOLE) sn = fmaf(lam_lo, s, sn);
          S[c][4 * r + u] = sn;
        }
      if (MODE != DS_SUMS) {
        const float qq[4] = {qc[r].x, qc[r].y, qc[r].z, qc[r].w};
#pragma unroll
        for (int c = 0; c < CPL; ++c)
#pragma unroll
          for (int u = 0; u < 4; ++u) o[c] = fmaf(S[c][4 * r + u], qq[u], o[c]);
      }
    }
    if (MODE != DS_SUMS) {
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        o[c] += __shfl_xor(o[c], 16, ME_WAVE);
        o[c] += __shfl_xor(o[c], 32, ME_WAVE);
        if (rg == 0 && has_col[c]) o32[((size_t)t * heads + head) * dv + col + c] = o[c];
      }
    }
  }
  if (MODE == DS_OUTPUTS) return;
#pragma unroll
  for (int c = 0; c < CPL; ++c)
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int i = rg * RPL + r;
      if (has_col[c] && i < d) srow[(size_t)i * dv + col + c] = S[c][r];
    }
}

// The states at the chunks' starts, in place of the chunks' sums: per item, head and element of the state,
// S = state[slot]; for each chunk of the item in order: (sum, place) = (place, S); S = decay^(chunk's tokens) * S + sum;
// state[slot] = S. Grid (elements / 256, head, item).
__global__ __launch_bounds__(256) void decay_state_chunk_starts_kernel(float* __restrict__ state, float* __restrict__ chunks,
                                                                        const float* __restrict__ decay,
                                                                        const int* __restrict__ item_start,
                                                                        const int* __restrict__ state_slots, int heads,
                                                                        int elements) {
  const int e = blockIdx.x * 256 + threadIdx.x, head = blockIdx.y, item = blockIdx.z;
  if (e >= elements) return;
  const int slot = state_slots[item];
  const int n = item_start[item + 1] - item_start[item];
  if (slot < 0 || n <= 0) return;
  int base = 0;
  for (int i = 0; i < item; ++i) base += (item_start[i + 1] - item_start[i] + DS_CHUNK - 1) / DS_CHUNK;
  const double lam = (double)decay[head] + (double)decay[heads + head];
  const int nc = (n + DS_CHUNK - 1) / DS_CHUNK, tail = n - (nc - 1) * DS_CHUNK;
  const float full = (float)pow(lam, (double)DS_CHUNK), last = (float)pow(lam, (double)tail);
  float* sp = state + ((size_t)slot * heads + head) * elements + e;
  float S = *sp;
  for (int c = 0; c < nc; ++c) {
    float* place = chunks + ((size_t)(base + c) * heads + head) * elements + e;
    const float sum = *place;
    *place = S;
    S = fmaf(c + 1 < nc ? full : last, S, sum);
  }
  *sp = S;
}

// ----------------------------------------------------------------------------------------------- finish
// One block per token. norm_kind 0: every head's dv outputs over their own sqrt(mean^2 + eps), no weight;
// 1: all heads' outputs together over sqrt(mean^2 + eps), times w [heads * dv]. Then times act(gate), where the gate
// is the last heads * dv columns of the projections.
template <typename T>
__global__ __launch_bounds__(1024) void decay_state_finish_kernel(const float* __restrict__ o32, const T* __restrict__ proj,
                                                                  int proj_cols, int gate_at, const float* __restrict__ w,
                                                                  T* __restrict__ out, int heads, int dv, int norm_kind,
                                                                  int gate_act, float eps) {
  __shared__ float inv[DS_MAX_D];  // per head (norm_kind 0: at most DS_MAX_D heads), or one value
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1), waves = blockDim.x / ME_WAVE;
  const int t = blockIdx.x, n = heads * dv;
  const float* orow = o32 + (size_t)t * n;
  if (norm_kind == 0) {
    for (int h = wave; h < heads; h += waves) {
      float ss = 0.f;
      for (int i = lane; i < dv; i += ME_WAVE) ss = fmaf(orow[h * dv + i], orow[h * dv + i], ss);
      ss = wave_sum(ss);
      if (lane == 0) inv[h] = rsqrtf(ss / (float)dv + eps);
    }
  } else {  // every wave adds up a stretch of the row, the stretches' sums are added in their order: the order of the
            // whole sum follows from the row's length and the block's size, which follows from the sizes too
    const int stretch = (n + waves - 1) / waves;
    float ss = 0.f;
    for (int i = wave * stretch + lane; i < min((wave + 1) * stretch, n); i += ME_WAVE) ss = fmaf(orow[i], orow[i], ss);
    ss = wave_sum(ss);
    if (lane == 0) inv[1 + wave] = ss;
    __syncthreads();
    if (threadIdx.x == 0) {
      float total = 0.f;
      for (int w = 0; w < waves; ++w) total += inv[1 + w];
      inv[0] = rsqrtf(total / (float)n + eps);
    }
  }
  __syncthreads();
  const T* gate = proj + (size_t)t * proj_cols + gate_at;
  T* dst = out + (size_t)t * n;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float y = orow[i] * (norm_kind == 0 ? inv[i / dv] : inv[0] * w[i]);
    y *= ds_act(to_float(gate[i]), gate_act);
    dst[i] = from_float<T>(y);
  }
}

// One instance of the scan: the chunked forms stage k (and q) in LDS, more than a launch may take without asking.
template <int RPL, int MODE, int CPL>
static int launch_scan(dim3 grid, hipStream_t stream, const float* q32, const float* k32, const float* v32, float* o32, float* state,
                       float* chunks, const float* decay, const int* item_start, const int* state_slots, int items, int heads,
                       int d, int dv) {
  const size_t lds = MODE == DS_WHOLE ? 0 : (size_t)(MODE == DS_OUTPUTS ? 2 : 1) * DS_CHUNK * 4 * (RPL + 4) * sizeof(float);
  static bool configured = false;
  if (lds > 48 * 1024 && !configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&decay_state_scan_kernel<RPL, MODE, CPL>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return me_fail("me_decay_state: %zu bytes of block memory are refused", lds);
    configured = true;
  }
  decay_state_scan_kernel<RPL, MODE, CPL><<<grid, 256, lds, stream>>>(q32, k32, v32, o32, state, chunks, decay, item_start,
                                                                      state_slots, items, heads, d, dv);
  return 0;
}

// --------------------------------------------------------------------------------------------- entry points
extern "C" int me_decay_state_padded_dim(int d) {  // the row length of the prepared q and k
  return d <= 32 ? 32 : d <= 64 ? 64 : d <= 128 ? 128 : 256;
}

// Bytes of float32 workspace that a step of `tokens` tokens in `items` items needs: prepared q, k, v, the raw outputs,
// and a state per chunk of 64 tokens (at most tokens / 64 + items of them) for steps that walk their chunks side by side.
extern "C" long long me_decay_state_workspace(long long tokens, long long items, int heads, int d, int dv) {
  const long long dp = me_decay_state_padded_dim(d);
  const long long chunks = tokens / DS_CHUNK + items;
  return tokens * heads * (2 * dp + 2 * (long long)dv) * 4 + chunks * heads * (long long)d * dv * 4 + 1024;
}

// proj [T, proj_cols]: q heads, k heads (d each), v heads, gate (dv each), so proj_cols = 2 heads (d + dv).
// decay: float32 [2, heads] (the decay's nearest float, then the rest of the configured value).
// state: float32 [slots, heads, d, dv]; item_start [items + 1], state_slots [items] (a negative slot: the item is skipped).
extern "C" int me_decay_state(const void* proj, const float* rope_table, int rd, int pairing, const int* positions,
                              const float* decay, const float* norm_w, float* state, const int* item_start,
                              const int* state_slots, void* out, void* workspace, int num_tokens, int items, int heads, int d,
                              int dv, int in_act, float key_scale, int norm_kind, int gate_act, float eps, int dtype,
                              int longest_item, hipStream_t stream) {
  if (num_tokens <= 0 || items <= 0) return 0;
  if (heads <= 0 || heads > DS_MAX_D || d <= 0 || d > DS_MAX_D || dv <= 0)
    return me_fail("me_decay_state: heads=%d d=%d dv=%d (heads and key size up to %d)", heads, d, dv, DS_MAX_D);
  if (rope_table && (rd <= 0 || rd > d || rd % 2 || (pairing & ~1)))
    return me_fail("me_decay_state: rotary_dim=%d with head size %d, pairing %d", rd, d, pairing);
  if (norm_kind != 0 && norm_kind != 1) return me_fail("me_decay_state: norm kind %d", norm_kind);
  if (norm_kind == 1 && !norm_w) return me_fail("me_decay_state: the norm over all heads needs its weight");
  if (items > 65535 || heads > 65535) return me_fail("me_decay_state: %d items, %d heads", items, heads);
  if ((uintptr_t)workspace & 15) return me_fail("me_decay_state: the workspace must be aligned to 16 bytes");
  const int dp = me_decay_state_padded_dim(d);
  const int proj_cols = 2 * heads * (d + dv);
  float* q32 = (float*)workspace;
  float* k32 = q32 + (size_t)num_tokens * heads * dp;
  float* v32 = k32 + (size_t)num_tokens * heads * dp;
  float* o32 = v32 + (size_t)num_tokens * heads * dv;
  const long long units = (long long)num_tokens * heads * 3;
  const unsigned prep_blocks = (unsigned)((units + 3) / 4);
  float* chunk_states = o32 + (size_t)num_tokens * heads * dv;
  // An item of more than two chunks (`longest_item`: the most tokens an item brings, 0 if unknown): all chunks of the
  // step side by side. Else every item in order, a block per item, head and 64 columns.
  const bool by_chunks = longest_item > 2 * DS_CHUNK;
  const int num_chunks = num_tokens / DS_CHUNK + items;  // an upper bound: blocks beyond the last chunk leave at once
  // two columns a lane where the rows a lane holds leave the registers for it and the heads are wide enough to fill the waves
  const int cpl = by_chunks && dp <= 128 && dv >= 32 ? 2 : 1;
  const dim3 scan_grid(by_chunks ? num_chunks : items, heads, (dv + 63) / 64);
  const dim3 scan_grid2(scan_grid.x, heads, (dv + 127) / 128);  // two columns a lane
  if (scan_grid.z > 65535 || (long long)d * dv > (1ll << 24)) return me_fail("me_decay_state: value heads of %d elements", dv);
  const dim3 starts_grid((d * dv + 255) / 256, heads, items);
  const int finish_threads = heads * dv >= 1024 * 2 && heads >= 16 ? 1024 : heads * dv >= 512 * 2 && heads >= 8 ? 512 : 256;
#define DS_SCAN_MODE(RPL, MODE)                                                                                              \
  do {                                                                                                                       \
    int failed;                                                                                                              \
    if (cpl == 2 && RPL <= 32 && MODE == DS_SUMS)                                                                            \
      failed = launch_scan<(RPL <= 32 ? RPL : 8), MODE, 2>(scan_grid2, stream, q32, k32, v32, o32, state, chunk_states, decay,  \
                                                           item_start, state_slots, items, heads, d, dv);                     \
    else                                                                                                                     \
      failed = launch_scan<RPL, MODE, 1>(scan_grid, stream, q32, k32, v32, o32, state, chunk_states, decay, item_start,         \
                                         state_slots, items, heads, d, dv);                                                   \
    if (failed) return failed;                                                                                               \
  } while (0)
#define DS_SCAN(RPL)                                                                                                         \
  do {                                                                                                                       \
    if (by_chunks) {                                                                                                         \
      DS_SCAN_MODE(RPL, DS_SUMS);                                                                                            \
      decay_state_chunk_starts_kernel<<<starts_grid, 256, 0, stream>>>(state, chunk_states, decay, item_start, state_slots,     \
                                                                       heads, d * dv);                                        \
      DS_SCAN_MODE(RPL, DS_OUTPUTS);                                                                                         \
    } else {                                                                                                                 \
      DS_SCAN_MODE(RPL, DS_WHOLE);                                                                                           \
    }                                                                                                                        \
  } while (0)
#define DS_RUN(T)                                                                                                           \
  do {                                                                                                                      \
    decay_state_prepare_kernel<T><<<prep_blocks, 256, 0, stream>>>((const T*)proj, proj_cols, rope_table, rd, pairing,        \
                                                                   positions, q32, k32, v32, num_tokens, heads, d, dp, dv,   \
                                                                   in_act, key_scale);                                       \
    if (dp == 32)                                                                                                           \
      DS_SCAN(8);                                                                                                           \
    else if (dp == 64)                                                                                                      \
      DS_SCAN(16);                                                                                                          \
    else if (dp == 128)                                                                                                     \
      DS_SCAN(32);                                                                                                          \
    else                                                                                                                    \
      DS_SCAN(64);                                                                                                          \
    /* a wave a head where a block can have that many: a head's sum is one trip to memory, not one per round of the waves */ \
    decay_state_finish_kernel<T><<<num_tokens, finish_threads, 0, stream>>>(o32, (const T*)proj, proj_cols, 2 * heads * d + heads * dv, \
                                                                 norm_w, (T*)out, heads, dv, norm_kind, gate_act, eps);      \
  } while (0)
  if (dtype == ME_F32)
    DS_RUN(float);
  else
    DS_RUN(bf16_t);
#undef DS_RUN
#undef DS_SCAN
#undef DS_SCAN_MODE
  return me_check_launch("me_decay_state");
}
