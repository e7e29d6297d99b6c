// Recurrent decode step of Taylor linear attention for gfx950 (HBM-bandwidth bound).
//
// One workgroup per (batch, head); one wavefront per 16 rows of the (dv x 273) fp32 state.
// A wavefront's 16 rows are 4368 contiguous floats = 1092 aligned float4, which it streams
// with fully coalesced 128-bit loads and stores (lane i of iteration t touches float4
// 64 t + i).  Since 256 floats per iteration < 273, an iteration touches at most two state
// rows and, after full unrolling, which two is a compile-time constant: partial dot
// products go to per-lane accumulators indexed by row, and one transposing butterfly at
// the end reduces all 16 rows across the wavefront.  phi(q) and phi(k) are expanded once
// per workgroup into LDS, in four copies shifted by 0..3 floats so that each lane's four
// consecutive features are one aligned 128-bit LDS read; the copies run 3 entries past 273
// and wrap, which is exactly where a float4 straddles into the next state row.
// The state is touched once per step and is far larger than any cache when every layer has its
// own: all 18 loads of a wavefront are non-temporal and leave at the top of the kernel, before
// the tables are built, and the stores are non-temporal too.
#include "common.hpp"

namespace based {

constexpr int kTabLen = 280;                     // 273 + 3 wrap entries, padded to 16 B multiple
constexpr int kRowsPerWave = 16;
constexpr int kVec4PerWave = kRowsPerWave * kExp / 4;  // 1092
constexpr int kIters = (kVec4PerWave + kWave - 1) / kWave;  // 18

__device__ __forceinline__ float phi_elem(const float* x, int f) {
  // TaylorExp element f of a 16-vector x: [1 | x/2 | x_i x_j / (4 sqrt 2)], row-major i,j.
  if (f == 0) return 1.0f;
  if (f <= kFeat) return x[f - 1] * 0.5f;
  int g = f - 1 - kFeat;
  return x[g >> 4] * x[g & 15] * 0.17677669529663687f;
}

template <typename T, int kMaxThreads>
__global__ __launch_bounds__(kMaxThreads) void lin_step_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    float* __restrict__ kv_state, float* __restrict__ k_state, T* __restrict__ y,
    int H, int dv, long q_sb, long q_sh, long k_sb, long k_sh, long v_sb, long v_sh,
    long y_sb, long y_sh, float eps) {
  __shared__ float s_x[2][kFeat];                            // [0] = k, [1] = q
  __shared__ __align__(16) float s_tab[2][4][kTabLen];       // [0] = phi(k), [1] = phi(q)
  __shared__ float s_v[1024];  // one entry per thread (the first dv are read)
  __shared__ float s_den;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const long bh = blockIdx.x;
  const int b = (int)(blockIdx.x / (unsigned)H), h = (int)(blockIdx.x % (unsigned)H);  // 32-bit: B * H < 2^31

  // State rows [16*wave, 16*wave+16) of this (b, h).  All of the wavefront's state is requested
  // before anything else: the loads depend on nothing but the workgroup's position, so the
  // HBM round trip runs under the set-up below (feature tables, two barriers).  The state is
  // touched exactly once per step and the whole batch's state is far larger than any cache:
  // non-temporal loads and stores keep it from displacing anything.
  // The small operands go first and nothing is loaded under a condition (a thread with nothing
  // to fetch re-reads a valid element): the wait for q, k and v can then leave the eighteen state
  // requests behind it in flight, and the feature tables are built under the HBM round trip
  // instead of after it.
  const int xi = tid & (2 * kFeat - 1);
  const T* x_src = (xi >> 4) ? (q + b * q_sb + h * q_sh) : (k + b * k_sb + h * k_sh);
  const float x_val = to_f32(x_src[xi & 15]);
  const float v_val = to_f32(v[b * v_sb + h * v_sh + (tid < dv ? tid : 0)]);
  // normaliser operands of wavefront 0 (every wavefront fetches them: no branch)
  constexpr int kNormIters = (kExp + kWave - 1) / kWave;  // 5
  float* ks = k_state + bh * kExp;
  float ks_old[kNormIters];
#pragma unroll
  for (int i = 0; i < kNormIters; ++i) {
    const int f = lane + kWave * i;
    ks_old[i] = ks[f < kExp ? f : 0];
  }

  f32x4* base = reinterpret_cast<f32x4*>(kv_state + (bh * dv + (long)kRowsPerWave * wave) * kExp);
  f32x4 d[kIters];
#pragma unroll
  for (int t = 0; t < kIters; ++t) {
    const int j = t * kWave + lane;
    d[t] = __builtin_nontemporal_load(base + (j < kVec4PerWave ? j : kVec4PerWave - 1));
  }

  // (stored by every thread, duplicates included: a load whose only use sits under a condition is
  // moved into that branch by the compiler, behind the state requests)
  s_x[xi >> 4][xi & 15] = x_val;
  s_v[tid] = v_val;
  __syncthreads();

  // Entry i of copy m holds feature e = i + m (features 273..275 wrap to 0..2, beyond that
  // zeros): a thread evaluates phi(k) and phi(q) once per e and files them in the four copies.
  for (int e = tid; e < kTabLen + 3; e += blockDim.x) {
    float val_k = 0.0f, val_q = 0.0f;
    if (e < kExp + 3) {
      const int f = e >= kExp ? e - kExp : e;
      val_k = phi_elem(s_x[0], f);
      val_q = phi_elem(s_x[1], f);
    }
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int i = e - m;
      if (i >= 0 && i < kTabLen) {
        s_tab[0][m][i] = val_k;
        s_tab[1][m][i] = val_q;
      }
    }
  }
  __syncthreads();

  // Normaliser: k_state += phi(k); den = phi(q) . k_state.  One wavefront owns it.
  if (wave == 0) {
    float part = 0.0f;
#pragma unroll
    for (int i = 0; i < kNormIters; ++i) {
      const int f = lane + kWave * i;
      if (f < kExp) {
        const float nk = ks_old[i] + s_tab[0][0][f];
        ks[f] = nk;
        part += s_tab[1][0][f] * nk;
      }
    }
    part = wave_sum(part);
    if (lane == 0) s_den = part;
  }

  // State rows [16*wave, 16*wave+16) of this (b, h).  v is wave-uniform: keep it scalar.
  float vrow[kRowsPerWave];
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r)
    vrow[r] = __builtin_bit_cast(
        float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, s_v[kRowsPerWave * wave + r])));

  float acc[kRowsPerWave];
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) acc[r] = 0.0f;

  const int e_lane = 4 * lane;
#pragma unroll
  for (int t = 0; t < kIters; ++t) {
    const int j = t * kWave + lane;
    const int rb = (256 * t) / kExp;              // first row touched by this iteration
    const int bnd = (rb + 1) * kExp - 256 * t;    // local element index where row rb+1 starts
    const bool two_rows = bnd < 256;
    if (t < kIters - 1 || j < kVec4PerWave) {
      const bool lane_hi = two_rows && (e_lane >= bnd);
      const int f0 = (256 * t - rb * kExp) + e_lane - (lane_hi ? kExp : 0);
      const int m = f0 & 3;
      const f32x4 pk = *reinterpret_cast<const f32x4*>(&s_tab[0][m][f0 - m]);
      const f32x4 pq = *reinterpret_cast<const f32x4*>(&s_tab[1][m][f0 - m]);
      const float v_lo = vrow[rb];
      const float v_hi = vrow[rb + 1 < kRowsPerWave ? rb + 1 : rb];
      f32x4 x = d[t];
      float s_lo = 0.0f, s_hi = 0.0f;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const bool hi = two_rows && (e_lane + c >= bnd);
        const float nv = __builtin_fmaf(hi ? v_hi : v_lo, pk[c], x[c]);
        x[c] = nv;
        const float p = pq[c] * nv;
        s_lo += hi ? 0.0f : p;
        s_hi += hi ? p : 0.0f;
      }
      d[t] = x;
      acc[rb] += s_lo;
      if (two_rows && rb + 1 < kRowsPerWave) acc[rb + 1] += s_hi;
    }
  }

  // The new state leaves in one piece per wavefront, after all of it has been read and updated:
  // 18 back-to-back stores of 1 KB instead of one store between every two loads' worth of
  // arithmetic (52.05 -> 51.09 us at B=128, alternating runs on one box: longer write bursts at
  // the memory).
#pragma unroll
  for (int t = 0; t < kIters; ++t) {
    const int j = t * kWave + lane;
    if (t < kIters - 1 || j < kVec4PerWave) __builtin_nontemporal_store(d[t], base + j);
  }

  // Transposing butterfly: 16 per-lane row sums -> lane l holds the total of row l >> 2.
#pragma unroll
  for (int half = 8, mask = 32; half >= 1; half >>= 1, mask >>= 1) {
    const bool up = (lane & mask) != 0;
#pragma unroll
    for (int i = 0; i < half; ++i) {
      const float a = acc[i], bb = acc[i + half];
      const float keep = up ? bb : a;
      const float send = up ? a : bb;
      acc[i] = keep + __shfl_xor(send, mask, 64);
    }
  }
  float num = acc[0];
  num += __shfl_xor(num, 2, 64);
  num += __shfl_xor(num, 1, 64);

  __syncthreads();
  if ((lane & 3) == 0) {
    const int e = kRowsPerWave * wave + (lane >> 2);
    y[b * y_sb + h * y_sh + e] = from_f32<T>(num / (s_den + eps));
  }
}


// ------------------------------------------------------------------------------------------
// The same step with the state update DEFERRED.  Writing the state back is half of the step's
// traffic; the output does not need it: with S the state as last written and (k_j, v_j) the tokens
// since then,
//   phi(q) . (S + sum_j phi(k_j) v_j^T) = phi(q) . S + sum_j (1 + s_j + s_j^2 / 2) v_j,  s_j = q . k_j / 4,
// so a step only READS the state and keeps the raw (k, v) of up to `period` - 1 tokens per
// (batch, head) in a small ring; every `period`-th step applies the whole ring and the current
// token in one pass (read, `period` rank-one updates, write).  k_state is small and is updated
// on every step.  The ring and its fill count live in device memory, per (batch, head), so that
// a recorded graph replays correctly (normally every workgroup of a call finds the same count, but
// nothing depends on it: a (batch, head) is one workgroup's business from the count to the state).
// ------------------------------------------------------------------------------------------
constexpr int kPendMax = BASED_DEFERRED_MAX_STEPS;

// Register budget: the kernel is left at what the allocator needs without spilling (192 vector
// registers at dv <= 64: two workgroups per compute unit).  Forcing three (launch bounds of three
// wavefronts per SIMD, 168 registers) makes the allocator spill 22 registers per lane to scratch
// memory, and the step is then a third slower instead of a tenth faster.
template <typename T, int kMaxThreads>
__global__ __launch_bounds__(kMaxThreads) void lin_step_deferred_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    float* __restrict__ kv_state, float* __restrict__ k_state, float* __restrict__ pend_k,
    float* __restrict__ pend_v, int* __restrict__ pend_n, T* __restrict__ y,
    int H, int dv, long q_sb, long q_sh, long k_sb, long k_sh, long v_sb, long v_sh,
    long y_sb, long y_sh, float eps, int period) {
  __shared__ float s_x[2][kFeat];                                   // [0] = k, [1] = q of this token
  __shared__ float s_v[1024];                                       // v of this token, one entry per thread
  __shared__ __align__(16) float s_tab[1 + kPendMax][4][kTabLen];   // [0] = phi(q); [1 + j] = phi(key j), applied steps only
  __shared__ float s_pk[kPendMax][kFeat];                           // keys 0..n-1 from the ring, key n = this token
  __shared__ float s_pv[kPendMax][256];                             // their values
  __shared__ float s_w[kPendMax];                                   // 1 + s_j + s_j^2 / 2
  __shared__ float s_den;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nthreads = blockDim.x;  // 4 dv
  const long bh = blockIdx.x;
  const int b = (int)(blockIdx.x / (unsigned)H), h = (int)(blockIdx.x % (unsigned)H);  // 32-bit: B * H < 2^31

  // small operands first, everything unconditional (see lin_step_kernel)
  int n = pend_n[bh];
  const int xi = tid & (2 * kFeat - 1);
  const T* x_src = (xi >> 4) ? (q + b * q_sb + h * q_sh) : (k + b * k_sb + h * k_sh);
  const float x_val = to_f32(x_src[xi & 15]);
  const float v_val = to_f32(v[b * v_sb + h * v_sh + (tid < dv ? tid : 0)]);
  constexpr int kNormIters = (kExp + kWave - 1) / kWave;  // 5
  float* ks = k_state + bh * kExp;
  float ks_old[kNormIters];
#pragma unroll
  for (int i = 0; i < kNormIters; ++i) {
    const int f = lane + kWave * i;
    ks_old[i] = ks[f < kExp ? f : 0];
  }
  // the ring: kPendMax x 16 keys (two loads cover it from 64 threads on), kPendMax x dv values
  // (= 2 x the number of threads)
  float* ring_k = pend_k + bh * (kPendMax * kFeat);
  float* ring_v = pend_v + bh * (long)kPendMax * dv;
  const int ki0 = tid & (kPendMax * kFeat - 1), ki1 = (tid + 64) & (kPendMax * kFeat - 1);
  const float rk0 = ring_k[ki0], rk1 = ring_k[ki1];
  const float rv0 = ring_v[tid], rv1 = ring_v[nthreads + tid];

  f32x4* base = reinterpret_cast<f32x4*>(kv_state + (bh * dv + (long)kRowsPerWave * wave) * kExp);
  f32x4 d[kIters];
#pragma unroll
  for (int t = 0; t < kIters; ++t) {
    const int j = t * kWave + lane;
    d[t] = __builtin_nontemporal_load(base + (j < kVec4PerWave ? j : kVec4PerWave - 1));
  }

  n = n < 0 ? 0 : (n > kPendMax - 1 ? kPendMax - 1 : n);   // tokens in the ring (a corrupt count cannot index outside it)
  const bool apply = n + 1 >= period;                  // this step writes the state
  const int n_keys = n + 1;                            // ring + this token

  s_x[xi >> 4][xi & 15] = x_val;
  s_v[tid] = v_val;
  s_pk[ki0 >> 4][ki0 & 15] = rk0;
  s_pk[ki1 >> 4][ki1 & 15] = rk1;
  {
    const int i0 = tid, i1 = nthreads + tid;  // < kPendMax * dv
    s_pv[i0 / dv][i0 % dv] = rv0;
    s_pv[i1 / dv][i1 % dv] = rv1;
  }
  __syncthreads();
  // this token takes slot n of the staged keys and values
  if (tid < kFeat) s_pk[n][tid] = s_x[0][tid];
  if (tid < dv) s_pv[n][tid] = s_v[tid];
  __syncthreads();

  // tables: phi(q) always; phi(key j) for the keys that are applied now
  const int n_tabs = apply ? 1 + n_keys : 1;
  for (int e = tid; e < n_tabs * (kTabLen + 3); e += nthreads) {
    const int tab = e / (kTabLen + 3), pos = e - tab * (kTabLen + 3);
    const float* src = tab == 0 ? s_x[1] : s_pk[tab - 1];
    float val = 0.0f;
    if (pos < kExp + 3) val = phi_elem(src, pos >= kExp ? pos - kExp : pos);
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int i = pos - m;
      if (i >= 0 && i < kTabLen) s_tab[tab][m][i] = val;
    }
  }
  // read-out weights of the keys (ring and this token)
  if (tid < n_keys) {
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < kFeat; ++i) s = __builtin_fmaf(s_x[1][i], s_pk[tid][i], s);
    s *= 0.25f;
    s_w[tid] = 1.0f + s + 0.5f * s * s;
  }
  __syncthreads();

  // Normaliser: k_state += phi(k); den = phi(q) . k_state.  One wavefront owns it.
  if (wave == 0) {
    float part = 0.0f;
#pragma unroll
    for (int i = 0; i < kNormIters; ++i) {
      const int f = lane + kWave * i;
      if (f < kExp) {
        const float nk = ks_old[i] + phi_elem(s_x[0], f);
        ks[f] = nk;
        part += s_tab[0][0][f] * nk;
      }
    }
    part = wave_sum(part);
    if (lane == 0) s_den = part;
  }

  float acc[kRowsPerWave];
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) acc[r] = 0.0f;

  const int e_lane = 4 * lane;
  const int row0 = kRowsPerWave * wave;
#pragma unroll
  for (int t = 0; t < kIters; ++t) {
    const int j = t * kWave + lane;
    const int rb = (256 * t) / kExp;              // first row touched by this iteration
    const int bnd = (rb + 1) * kExp - 256 * t;    // local element index where row rb+1 starts
    const bool two_rows = bnd < 256;
    const int rb1 = rb + 1 < kRowsPerWave ? rb + 1 : rb;
    if (t < kIters - 1 || j < kVec4PerWave) {
      const bool lane_hi = two_rows && (e_lane >= bnd);
      const int f0 = (256 * t - rb * kExp) + e_lane - (lane_hi ? kExp : 0);
      const int m = f0 & 3;
      const f32x4 pq = *reinterpret_cast<const f32x4*>(&s_tab[0][m][f0 - m]);
      f32x4 x = d[t];
      if (apply) {
#pragma unroll 1
        for (int kk = 0; kk < n_keys; ++kk) {
          const f32x4 pk = *reinterpret_cast<const f32x4*>(&s_tab[1 + kk][m][f0 - m]);
          const float v_lo = s_pv[kk][row0 + rb], v_hi = s_pv[kk][row0 + rb1];
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const bool hi = two_rows && (e_lane + c >= bnd);
            x[c] = __builtin_fmaf(hi ? v_hi : v_lo, pk[c], x[c]);
          }
        }
        __builtin_nontemporal_store(x, base + j);
      }
      float s_lo = 0.0f, s_hi = 0.0f;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const bool hi = two_rows && (e_lane + c >= bnd);
        const float p = pq[c] * x[c];
        s_lo += hi ? 0.0f : p;
        s_hi += hi ? p : 0.0f;
      }
      acc[rb] += s_lo;
      if (two_rows && rb + 1 < kRowsPerWave) acc[rb + 1] += s_hi;
    }
  }

  // Transposing butterfly: 16 per-lane row sums -> lane l holds the total of row l >> 2.
#pragma unroll
  for (int half = 8, mask = 32; half >= 1; half >>= 1, mask >>= 1) {
    const bool up = (lane & mask) != 0;
#pragma unroll
    for (int i = 0; i < half; ++i) {
      const float a = acc[i], bb = acc[i + half];
      const float keep = up ? bb : a;
      const float send = up ? a : bb;
      acc[i] = keep + __shfl_xor(send, mask, 64);
    }
  }
  float num = acc[0];
  num += __shfl_xor(num, 2, 64);
  num += __shfl_xor(num, 1, 64);

  const int e_out = row0 + (lane >> 2);
  if (!apply) {
    // the state as read lacks the ring's tokens and this one: their share of the read-out
    float extra = 0.0f;
#pragma unroll 1
    for (int kk = 0; kk < n_keys; ++kk) extra = __builtin_fmaf(s_w[kk], s_pv[kk][e_out], extra);
    num += extra;
  }

  __syncthreads();
  if ((lane & 3) == 0) y[b * y_sb + h * y_sh + e_out] = from_f32<T>(num / (s_den + eps));

  // the ring takes this token, or starts again after the state was written
  if (!apply) {
    if (tid < kFeat) ring_k[n * kFeat + tid] = s_x[0][tid];
    if (tid < dv) ring_v[(long)n * dv + tid] = s_v[tid];
  }
  if (tid == 0) pend_n[bh] = apply ? 0 : n + 1;
}

// Brings kv_state up to date without a new token: S += sum over the ring of phi(k_j) v_j^T, ring
// emptied.  Not a performance path (checkpointing, inspection, leaving the deferred mode).
__global__ __launch_bounds__(256) void lin_flush_deferred_kernel(float* __restrict__ kv_state,
                                                                 const float* __restrict__ pend_k,
                                                                 const float* __restrict__ pend_v,
                                                                 int* __restrict__ pend_n, int dv) {
  __shared__ float s_pk[kPendMax][kFeat];
  __shared__ float s_pv[kPendMax][256];
  const long bh = blockIdx.x;
  int n = pend_n[bh];
  n = n < 0 ? 0 : (n > kPendMax - 1 ? kPendMax - 1 : n);
  for (int i = threadIdx.x; i < kPendMax * kFeat; i += blockDim.x) s_pk[i >> 4][i & 15] = pend_k[bh * (kPendMax * kFeat) + i];
  for (int i = threadIdx.x; i < kPendMax * dv; i += blockDim.x) s_pv[i / dv][i % dv] = pend_v[bh * (long)kPendMax * dv + i];
  __syncthreads();
  if (n > 0) {
    float* st = kv_state + bh * (long)dv * kExp;
    for (int idx = threadIdx.x; idx < dv * kExp; idx += blockDim.x) {
      const int e = idx / kExp, f = idx - e * kExp;
      float x = st[idx];
      for (int j = 0; j < n; ++j) x = __builtin_fmaf(s_pv[j][e], phi_elem(s_pk[j], f), x);
      st[idx] = x;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) pend_n[bh] = 0;
}

}  // namespace based

extern "C" BASED_API int based_linear_attn_step(const void* q, const void* k, const void* v,
                                      float* kv_state, float* k_state, void* y,
                                      int64_t B, int64_t H, int64_t dv,
                                      int64_t q_sb, int64_t q_sh, int64_t k_sb, int64_t k_sh,
                                      int64_t v_sb, int64_t v_sh, int64_t y_sb, int64_t y_sh,
                                      float eps, int io_dtype, void* stream) {
  using namespace based;
  BASED_REQUIRE(q && k && v && kv_state && k_state && y, BASED_ERR_ARG,
                "linear_attn_step: null pointer argument");
  BASED_REQUIRE(B >= 0 && H > 0, BASED_ERR_ARG, "linear_attn_step: bad sizes B=%ld H=%ld",
                (long)B, (long)H);
  BASED_REQUIRE(dv >= 16 && dv <= 256 && dv % 16 == 0, BASED_ERR_SHAPE,
                "linear_attn_step: head dim %ld unsupported (multiple of 16 in [16, 256])", (long)dv);
  BASED_REQUIRE((reinterpret_cast<uintptr_t>(kv_state) & 15) == 0, BASED_ERR_ALIGN,
                "linear_attn_step: kv_state must be 16-byte aligned");
  BASED_REQUIRE(io_dtype == BASED_BF16 || io_dtype == BASED_F32, BASED_ERR_DTYPE,
                "linear_attn_step: io_dtype %d unsupported", io_dtype);
  BASED_REQUIRE(B * H < (1ll << 31), BASED_ERR_SHAPE, "linear_attn_step: B*H too large");
  if (B == 0) return BASED_OK;
  dim3 grid((unsigned)(B * H)), block((unsigned)(dv / 16 * 64));
  hipStream_t s = static_cast<hipStream_t>(stream);
#define BASED_LAUNCH_STEP(T, MAXT)                                                              \
  hipLaunchKernelGGL((lin_step_kernel<T, MAXT>), grid, block, 0, s, (const T*)q, (const T*)k,   \
                     (const T*)v, kv_state, k_state, (T*)y, (int)H, (int)dv, q_sb, q_sh, k_sb,  \
                     k_sh, v_sb, v_sh, y_sb, y_sh, eps)
  // The register budget follows the workgroup size: 4 waves (dv <= 64) may use 256 VGPRs.
  if (io_dtype == BASED_BF16) {
    if (dv <= 64) BASED_LAUNCH_STEP(__bf16, 256);
    else if (dv <= 128) BASED_LAUNCH_STEP(__bf16, 512);
    else BASED_LAUNCH_STEP(__bf16, 1024);
  } else {
    if (dv <= 64) BASED_LAUNCH_STEP(float, 256);
    else if (dv <= 128) BASED_LAUNCH_STEP(float, 512);
    else BASED_LAUNCH_STEP(float, 1024);
  }
#undef BASED_LAUNCH_STEP
  return check_launch("linear_attn_step");
}

extern "C" BASED_API int based_linear_attn_step_deferred(
    const void* q, const void* k, const void* v, float* kv_state, float* k_state, float* pend_k, float* pend_v,
    int32_t* pend_n, void* y, int64_t B, int64_t H, int64_t dv, int64_t q_sb, int64_t q_sh, int64_t k_sb,
    int64_t k_sh, int64_t v_sb, int64_t v_sh, int64_t y_sb, int64_t y_sh, float eps, int period, int io_dtype,
    void* stream) {
  using namespace based;
  BASED_REQUIRE(q && k && v && kv_state && k_state && pend_k && pend_v && pend_n && y, BASED_ERR_ARG,
                "linear_attn_step_deferred: null pointer argument");
  BASED_REQUIRE(B >= 0 && H > 0, BASED_ERR_ARG, "linear_attn_step_deferred: bad sizes B=%ld H=%ld", (long)B, (long)H);
  BASED_REQUIRE(dv >= 16 && dv <= 256 && dv % 16 == 0, BASED_ERR_SHAPE,
                "linear_attn_step_deferred: head dim %ld unsupported (multiple of 16 in [16, 256])", (long)dv);
  BASED_REQUIRE(period >= 1 && period <= kPendMax, BASED_ERR_ARG,
                "linear_attn_step_deferred: period %d outside [1, %d]", period, kPendMax);
  BASED_REQUIRE((reinterpret_cast<uintptr_t>(kv_state) & 15) == 0, BASED_ERR_ALIGN,
                "linear_attn_step_deferred: kv_state must be 16-byte aligned");
  BASED_REQUIRE(io_dtype == BASED_BF16 || io_dtype == BASED_F32, BASED_ERR_DTYPE,
                "linear_attn_step_deferred: io_dtype %d unsupported", io_dtype);
  BASED_REQUIRE(B * H < (1ll << 31), BASED_ERR_SHAPE, "linear_attn_step_deferred: B*H too large");
  if (B == 0) return BASED_OK;
  dim3 grid((unsigned)(B * H)), block((unsigned)(dv / 16 * 64));
  hipStream_t s = static_cast<hipStream_t>(stream);
#define BASED_LAUNCH_STEP(T, MAXT)                                                                        \
  hipLaunchKernelGGL((lin_step_deferred_kernel<T, MAXT>), grid, block, 0, s, (const T*)q, (const T*)k,    \
                     (const T*)v, kv_state, k_state, pend_k, pend_v, pend_n, (T*)y, (int)H, (int)dv,      \
                     q_sb, q_sh, k_sb, k_sh, v_sb, v_sh, y_sb, y_sh, eps, period)
  if (io_dtype == BASED_BF16) {
    if (dv <= 64) BASED_LAUNCH_STEP(__bf16, 256);
    else if (dv <= 128) BASED_LAUNCH_STEP(__bf16, 512);
    else BASED_LAUNCH_STEP(__bf16, 1024);
  } else {
    if (dv <= 64) BASED_LAUNCH_STEP(float, 256);
    else if (dv <= 128) BASED_LAUNCH_STEP(float, 512);
    else BASED_LAUNCH_STEP(float, 1024);
  }
#undef BASED_LAUNCH_STEP
  return check_launch("linear_attn_step_deferred");
}

extern "C" BASED_API int based_linear_attn_flush_deferred(float* kv_state, const float* pend_k, const float* pend_v,
                                                          int32_t* pend_n, int64_t B, int64_t H, int64_t dv,
                                                          void* stream) {
  using namespace based;
  BASED_REQUIRE(kv_state && pend_k && pend_v && pend_n, BASED_ERR_ARG, "linear_attn_flush_deferred: null pointer argument");
  BASED_REQUIRE(B >= 0 && H > 0 && B * H < (1ll << 31), BASED_ERR_ARG, "linear_attn_flush_deferred: bad sizes");
  BASED_REQUIRE(dv >= 16 && dv <= 256 && dv % 16 == 0, BASED_ERR_SHAPE,
                "linear_attn_flush_deferred: head dim %ld unsupported (multiple of 16 in [16, 256])", (long)dv);
  if (B == 0) return BASED_OK;
  hipLaunchKernelGGL(lin_flush_deferred_kernel, dim3((unsigned)(B * H)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     kv_state, pend_k, pend_v, pend_n, (int)dv);
  return check_launch("linear_attn_flush_deferred");
}
