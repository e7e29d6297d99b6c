// Projections of a single-token step for gfx950: y[M, N] = pro(x)[M, K] . W[N, K]^T (+ bias) for
// M <= 32 rows (the decoding batch, walked 8 at a time), bf16 in and out, fp32 accumulation.
//
// At these sizes a projection is a read of its weight matrix (2 .. 8 MB, 100 MB for the LM head)
// and nothing else: a tiled GEMM leaves the machine idle and costs 6 - 17 us of launch + tail
// latency.  Here ONE wavefront owns R consecutive weight rows over the WHOLE contraction length:
// a lane fetches 16-byte pieces p = lane + 64 c (c < C chunks) of every row, so that a row is
// read as contiguous 1 KB requests, multiplies them with its pieces of the M activation rows
// (held in registers for the lifetime of the wavefront) by `v_dot2_f32_bf16`, and the R x M
// partial sums are added up across the 64 lanes by a halving tree (row-pair swaps, then DPP
// rotations).  The weight rows of the next row group are requested before the current group is
// multiplied.
//
// Because every workgroup sees whole activation rows, the element-wise operation in front of the
// projection is evaluated inside it (once per workgroup of 4 or 8 wavefronts, shared through LDS)
// instead of by a launch of its own:
//   * residual add + RMSNorm (block.py:134-139,151-155 + layer_norm.py:117-118): every
//     workgroup forms r = x + residual and its norm; workgroup 0 writes r out for the next block;
//     the rows of x can be gathered through an index (the token embedding lookup of the first
//     block);
//   * the SwiGLU gate between fc1 and fc2 (mlp.py:147-151).
// What FOLLOWS a projection whose output is consumed in (value, gate) pairs runs in its tail: a
// wavefront then takes R/2 rows of the value half of the weight and the R/2 matching rows of the
// gate half, so that after the sums one lane holds both numbers of an output element, and
//   * the SwiGLU gate after fc1 (mlp.py:147-151), or
//   * the step of the gated short convolution after BaseConv's in_proj (convolution.py:78-109,
//     195-210: roll the (B, D, K) state, convolve, SiLU, gate), whose state element has exactly
//     one owner here,
// is applied to the bf16-rounded pair before anything is stored.
// All of them use the arithmetic (and the roundings to bf16) of the stand-alone kernels.
#include "common.hpp"

namespace based {

struct DecodeLinearArgs {
  const __bf16* x;
  long x_sr;
  const int64_t* x_index;  // nullptr, or row m of x is x[x_index[m] * x_sr]
  long x_index_rows;
  const __bf16* w;
  long w_sr;
  const __bf16* bias;
  __bf16* y;
  long y_sr;
  int M, N, K;
  const float* res_in;
  long ri_sr;
  float* res_out;
  long ro_sr;
  const __bf16* norm_w;
  float eps;
  int n_groups;
  // paired epilogues: F = N / 2 outputs
  void* conv_state;  // (rows, F, conv_k), rows counted from the first row of the whole call
  const __bf16* conv_w;
  const __bf16* conv_b;
  int conv_k, conv_state_f32, m0;
};

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// Where a load has nothing to fetch (a piece past the end of a row, an absent bias or residual) it
// is pointed at these instead of being skipped or having its result replaced: a load under a
// branch, or one whose result feeds a select, is waited for on the spot, and the memory round
// trips of a wavefront then run one after the other instead of together.
// (Not declared const: constant data lives in another address space, and a pointer that may be
// either turns every load through it into a flat one, which is waited for like a branch.)
__device__ __attribute__((aligned(64))) uint32_t kZeroPage[16] = {};
__device__ __attribute__((aligned(16))) uint32_t kNanPage[4] = {0x7fc07fc0u, 0x7fc07fc0u, 0x7fc07fc0u, 0x7fc07fc0u};

__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
}

template <int CTRL> __device__ __forceinline__ float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false);
  return v + __builtin_bit_cast(float, moved);
}

// Sums each of the N per-lane values over the 64 lanes.  On return, out[j] of a lane in 16-lane
// row w (w = lane / 16) is the total of v[4 j + 2 (w & 1) + (w >> 1)], the same in all 16 lanes.
template <int N> __device__ __forceinline__ void reduce_tree(const float (&v)[N], float (&out)[N / 4]) {
  float half[N / 2];
#pragma unroll
  for (int i = 0; i < N / 2; ++i) {
    // Lanes 32..63 of a trade places with lanes 0..31 of b.  Inline assembly: the compiler's
    // builtin returns the same register for both results here.  A vector instruction must not
    // read the result of a dot-product instruction in the three issue slots after it (two after
    // other vector instructions); the compiler cannot see into the assembly and the sums come
    // straight from v_dot2, hence the s_nop.
    float a = v[2 * i], b = v[2 * i + 1];
    asm volatile("s_nop 3\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    half[i] = a + b;
  }
#pragma unroll
  for (int j = 0; j < N / 4; ++j) {
    // odd 16-lane rows of a trade places with the even rows of b
    float a = half[2 * j], b = half[2 * j + 1];
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    float s = a + b;
    s = dpp_add<0x128>(s);  // row_ror:8
    s = dpp_add<0x124>(s);  // row_ror:4
    s = dpp_add<0x122>(s);  // row_ror:2
    s = dpp_add<0x121>(s);  // row_ror:1
    out[j] = s;
  }
}

// Total over the 64 lanes in every lane, with the pairing of the xor butterfly 32, 16, 8, 4, 2, 1
// (after each step the values repeat with that period, so a rotation by k within a 16-lane row
// reaches a lane that holds what lane ^ k holds): the same bits as `wave_sum`, without the LDS
// crossbar.
__device__ __forceinline__ float wave_sum_dpp(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  x = a + b;
  a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  x = a + b;
  x = dpp_add<0x128>(x);
  x = dpp_add<0x124>(x);
  x = dpp_add<0x122>(x);
  x = dpp_add<0x121>(x);
  return x;
}

__device__ __forceinline__ float silu_f(float a) { return a / (1.0f + __expf(-a)); }

enum { kProNone = BASED_PROLOGUE_NONE, kProNorm = BASED_PROLOGUE_ADD_RMS_NORM, kProSwiglu = BASED_PROLOGUE_SWIGLU };
enum { kEpiNone = BASED_EPILOGUE_NONE, kEpiSwiglu = BASED_EPILOGUE_SWIGLU, kEpiConv = BASED_EPILOGUE_GATED_CONV_STEP };

__device__ __forceinline__ void lds_barrier() {
  // the waves only exchange data through LDS here; a fence over global memory as well would wait
  // for the weight rows that are still on their way
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// C: 512-element chunks of the contraction length a lane holds (K <= 512 C); MT: activation rows
// held (M <= MT); a row group is R = 8 / C weight rows, one per wavefront at a time.  A prologue
// is evaluated ONCE per workgroup (norm: wavefront w owns rows w, w + 4; gate: the (row, chunk)
// pieces are dealt round the wavefronts) and the packed bf16 rows go to all its wavefronts
// through LDS.
// Wavefronts per workgroup: four share a prologue (with eight, one per row of the larger tile, a
// 4096-row projection is 128 workgroups and leaves half the compute units idle: 6.7 against
// 6.1 us at 8 rows); without a prologue nothing is shared and single wavefronts spread over the
// most compute units.
// One tile of at most MT activation rows (a.M of them, starting at row a.m0 of the call; the
// pointers in `a` already point at the tile).
template <int C, int MT, int PRO, int EPI>
__device__ __forceinline__ void decode_linear_tile(const DecodeLinearArgs& a, bool first_tile) {
  constexpr int WV = PRO == kProNone ? 1 : 4;
  constexpr int R = 8 / C;
  constexpr int RH = R / 2;  // paired epilogues: RH value rows + RH gate rows per group
  static_assert(EPI == kEpiNone || R >= 2, "a paired epilogue needs two rows per group");
  const int F = a.N / 2;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int e0[C];
  bool live[C];
#pragma unroll
  for (int c = 0; c < C; ++c) {
    const int e = (c * 64 + lane) * 8;
    live[c] = e < a.K;
    e0[c] = live[c] ? e : 0;
  }
  const __bf16* zeros = reinterpret_cast<const __bf16*>(kZeroPage);

  auto load_rows = [&](int g, u32x4 (&dst)[R][C]) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      int row = g * R + r;
      bool ok = row < a.N;
      if constexpr (EPI != kEpiNone) {
        const int f = g * RH + (r < RH ? r : r - RH);
        row = r < RH ? f : F + f;
        ok = f < F;
      }
      // rows past the end are never stored and pieces past the end of a row meet zeros from the
      // activations: both are simply fetched from a valid address
      const __bf16* src = a.w + (long)(ok ? row : 0) * a.w_sr;
#pragma unroll
      for (int c = 0; c < C; ++c) dst[r][c] = *reinterpret_cast<const u32x4*>(src + e0[c]);
    }
  };
  // row m of the activations (rows past M are never stored: any valid row will do); a row whose
  // index is out of range reads as NaN
  auto x_row = [&](int m, bool& poison) -> const __bf16* {
    m = m < a.M ? m : 0;
    long src = m;
    poison = false;
    if (a.x_index != nullptr) {
      src = a.x_index[m];
      poison = src < 0 || src >= a.x_index_rows;
      if (poison) src = 0;
    }
    return a.x + src * a.x_sr;
  };
  const __bf16* nans = reinterpret_cast<const __bf16*>(kNanPage);

  const int n_wg = gridDim.x, wg = blockIdx.x;
  int g = wg * WV + wave;
  const int g_step = n_wg * WV;
  const bool have = g < a.n_groups;
  u32x4 wcur[R][C];
  load_rows(have ? g : 0, wcur);  // in flight while the activations are prepared

  // ---- activations: packed bf16 pieces of every row.  Without a prologue every wavefront fetches
  // them itself (measured faster than sharing them); a prologue is evaluated once per workgroup
  // and handed round through LDS ----
  u32x4 xr[MT][C];
  if constexpr (PRO == kProNone) {
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      bool poison;
      const __bf16* xrow = x_row(m, poison);
#pragma unroll
      for (int c = 0; c < C; ++c)
        xr[m][c] = *reinterpret_cast<const u32x4*>(live[c] ? (poison ? nans : xrow + e0[c]) : zeros);
    }
  } else {
  __shared__ u32x4 xs[MT][C][64];
  if (!first_tile) lds_barrier();  // every wavefront has taken the previous tile out of LDS
  if constexpr (PRO == kProNorm) {
#pragma unroll
    for (int m = wave; m < MT; m += WV)
    if (m < a.M) {
      bool poison;
      const __bf16* xrow = x_row(m, poison);
      float v[C][8];
      float ss = 0.f;
      bf16x8 nw[C];
      const bool has_res = a.res_in != nullptr;
#pragma unroll
      for (int c = 0; c < C; ++c) {
        const bf16x8 h = *reinterpret_cast<const bf16x8*>(live[c] ? xrow + e0[c] : zeros);
        nw[c] = *reinterpret_cast<const bf16x8*>(live[c] ? a.norm_w + e0[c] : zeros);
        const float* rp = has_res && live[c] ? a.res_in + (long)m * a.ri_sr + e0[c] : reinterpret_cast<const float*>(kZeroPage);
        const f32x4 r0 = reinterpret_cast<const f32x4*>(rp)[0], r1 = reinterpret_cast<const f32x4*>(rp)[1];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[c][i] = to_f32(h[i]) + r0[i];
          v[c][4 + i] = to_f32(h[4 + i]) + r1[i];
        }
      }
#pragma unroll
      for (int c = 0; c < C; ++c) {
        if (a.res_out != nullptr && wg == 0 && live[c]) {
          float* op = a.res_out + (long)m * a.ro_sr + e0[c];
          reinterpret_cast<f32x4*>(op)[0] = f32x4{v[c][0], v[c][1], v[c][2], v[c][3]};
          reinterpret_cast<f32x4*>(op)[1] = f32x4{v[c][4], v[c][5], v[c][6], v[c][7]};
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          v[c][i] = to_f32(from_f32<__bf16>(v[c][i]));  // the norm sees the sum in bf16
          ss = __builtin_fmaf(v[c][i], v[c][i], ss);
        }
      }
      ss = wave_sum_dpp(ss);
      float rstd = rsqrtf(ss / (float)a.K + a.eps);
      if (poison) rstd = __builtin_nanf("");
#pragma unroll
      for (int c = 0; c < C; ++c) {
        float o[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = v[c][i] * rstd * to_f32(nw[c][i]);
        xs[m][c][lane] = u32x4{pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]), pack_bf16(o[4], o[5]), pack_bf16(o[6], o[7])};
      }
    }
  } else {
    // the (row, chunk) pieces are dealt round the wavefronts
    for (int item = wave; item < a.M * C; item += WV) {
      const int m = item / C, c = item % C;
      const int e = (c * 64 + lane) * 8;
      const bool in_row = e < a.K;
      bool poison;
      const __bf16* xrow = x_row(m, poison);
      const bf16x8 val = *reinterpret_cast<const bf16x8*>(in_row ? (poison ? nans : xrow + e) : zeros);
      const bf16x8 gate = *reinterpret_cast<const bf16x8*>(in_row ? xrow + a.K + e : zeros);
      float o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float sg = to_f32(from_f32<__bf16>(silu_f(to_f32(gate[i]))));  // as the stand-alone gate kernel
        o[i] = to_f32(val[i]) * sg;
      }
      xs[m][c][lane] = u32x4{pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]), pack_bf16(o[4], o[5]), pack_bf16(o[6], o[7])};
    }
  }
  lds_barrier();
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int c = 0; c < C; ++c) xr[m][c] = xs[m < a.M ? m : 0][c][lane];
  }
  if (!have) return;

  // ---- row groups ----
  // Which output this lane stores is fixed by the reduction tree: lane j of 16-lane row w ends up
  // with sum 4 j + 2 (w & 1) + (w >> 1), sums being numbered r * MT + m.
  constexpr int kOwners = (EPI == kEpiNone ? R : RH) * MT / 4;
  const int w16 = lane >> 4, j16 = lane & 15;
  const int own_idx = 4 * j16 + 2 * (w16 & 1) + (w16 >> 1);
  const int own_r = own_idx / MT, own_m = own_idx % MT;
  // one row group: products, sums across the lanes, tail, store
  auto finish_group = [&](const u32x4 (&wcur)[R][C], int g) {
    // what the tail needs from memory is asked for before the products, not after the sums
    const int out_col = EPI == kEpiNone ? g * R + own_r : g * RH + own_r;
    const bool owner = j16 < kOwners && own_m < a.M && out_col < (EPI == kEpiNone ? a.N : F);
    const int col_c = owner ? out_col : 0;
    const bool has_bias = a.bias != nullptr;
    const float bias_v = to_f32(*(has_bias ? a.bias + col_c : zeros));
    float bias_g = 0.f;
    if constexpr (EPI != kEpiNone) bias_g = to_f32(*(has_bias ? a.bias + F + col_c : zeros));
    float st[4] = {0.f, 0.f, 0.f, 0.f}, cw[4] = {0.f, 0.f, 0.f, 0.f}, cb = 0.f;
    long st_base = 0;
    if constexpr (EPI == kEpiConv) {
      st_base = ((long)(a.m0 + (owner ? own_m : 0)) * F + col_c) * a.conv_k;
      const float* s32 = reinterpret_cast<const float*>(a.conv_state) + st_base;
      const __bf16* s16 = reinterpret_cast<const __bf16*>(a.conv_state) + st_base;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool in_state = j + 1 < a.conv_k;  // rolled by one on the way in
        const float f32v = *(in_state && a.conv_state_f32 ? s32 + j + 1 : reinterpret_cast<const float*>(kZeroPage));
        const float f16v = to_f32(*(in_state && !a.conv_state_f32 ? s16 + j + 1 : zeros));
        st[j] = f32v + f16v;  // one of the two is the zero page
        cw[j] = to_f32(*(j < a.conv_k ? a.conv_w + (long)col_c * a.conv_k + j : zeros));
      }
      cb = to_f32(*(a.conv_b != nullptr ? a.conv_b + col_c : zeros));
    }

    float acc[R * MT];
#pragma unroll
    for (int i = 0; i < R * MT; ++i) acc[i] = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int c = 0; c < C; ++c)
#pragma unroll
        for (int d = 0; d < 4; ++d)
#pragma unroll
          for (int m = 0; m < MT; ++m) acc[r * MT + m] = dot2_bf16(wcur[r][c][d], xr[m][c][d], acc[r * MT + m]);

    float tot[R * MT / 4];
    reduce_tree<R * MT>(acc, tot);
    if constexpr (EPI == kEpiNone) {
      float mine = 0.f;
#pragma unroll
      for (int j = 0; j < kOwners; ++j) mine = (j16 == j) ? tot[j] : mine;
      if (owner) a.y[(long)own_m * a.y_sr + out_col] = from_f32<__bf16>(mine + bias_v);
    } else {
      // value (r, m) and gate (r, m) are RH * MT sums apart: the same lane, kOwners slots on
      float val = 0.f, gate = 0.f;
#pragma unroll
      for (int j = 0; j < kOwners; ++j) {
        val = (j16 == j) ? tot[j] : val;
        gate = (j16 == j) ? tot[j + kOwners] : gate;
      }
      if (owner) {
        // the pair as the projection alone would have stored it
        val = to_f32(from_f32<__bf16>(val + bias_v));
        gate = to_f32(from_f32<__bf16>(gate + bias_g));
        float out;
        if constexpr (EPI == kEpiSwiglu) {
          out = val * to_f32(from_f32<__bf16>(silu_f(gate)));
        } else {
          // one step of the gated short convolution on channel out_col of sequence m0 + own_m
          float accum = cb;
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (j < a.conv_k) {
              if (j + 1 == a.conv_k) st[j] = val;
              accum = __builtin_fmaf(cw[j], st[j], accum);
              if (a.conv_state_f32)
                reinterpret_cast<float*>(a.conv_state)[st_base + j] = st[j];
              else
                reinterpret_cast<__bf16*>(a.conv_state)[st_base + j] = from_f32<__bf16>(st[j]);
            }
          out = silu_f(accum) * gate;
        }
        a.y[(long)own_m * a.y_sr + out_col] = from_f32<__bf16>(out);
      }
    }
  };

  if (g_step >= a.n_groups) {  // one round (all but the LM head)
    finish_group(wcur, g);
    return;
  }
  // Several rounds: the rows of the next group are requested before the current one is worked
  // on, into a second set of registers (the two sets take turns, nothing is copied), and always
  // (past the end: the current group again), so that the number of loads in flight is the same on
  // every path and the wait before the products can leave exactly those outstanding.
  u32x4 wother[R][C];
  for (;;) {
    const int g1 = g + g_step;
    const bool more1 = g1 < a.n_groups;
    load_rows(more1 ? g1 : g, wother);
    finish_group(wcur, g);
    if (!more1) break;
    const int g2 = g1 + g_step;
    const bool more2 = g2 < a.n_groups;
    load_rows(more2 ? g2 : g1, wcur);
    finish_group(wother, g1);
    if (!more2) break;
    g = g2;
  }
}

// More than MT rows: the tiles are walked inside the launch (the weight rows of a wavefront come
// from its own L1 / L2 from the second tile on).
template <int C, int MT, int PRO, int EPI>
__global__ __launch_bounds__(PRO == kProNone ? 64 : 256) void decode_linear_kernel(const DecodeLinearArgs a) {
  if (a.M <= MT) {
    decode_linear_tile<C, MT, PRO, EPI>(a, true);
    return;
  }
  for (int m0 = 0; m0 < a.M; m0 += MT) {
    DecodeLinearArgs t = a;
    t.M = a.M - m0 < MT ? a.M - m0 : MT;
    t.m0 = m0;
    if (a.x_index != nullptr)
      t.x_index = a.x_index + m0;
    else
      t.x = a.x + (long)m0 * a.x_sr;
    t.y = a.y + (long)m0 * a.y_sr;
    if (a.res_in != nullptr) t.res_in = a.res_in + (long)m0 * a.ri_sr;
    if (a.res_out != nullptr) t.res_out = a.res_out + (long)m0 * a.ro_sr;
    decode_linear_tile<C, MT, PRO, EPI>(t, m0 == 0);
  }
}

constexpr int kDecodeLinearMaxWaves = 4096;  // row groups beyond this many are walked in a loop

template <int C, int MT, int EPI>
void launch_decode_linear_pro(const DecodeLinearArgs& a, int prologue, hipStream_t s) {
  const int wv = prologue == kProNone ? 1 : 4;  // WV of the kernel
  const int n_wg = (a.n_groups + wv - 1) / wv, cap = kDecodeLinearMaxWaves / wv;
  const dim3 grid((unsigned)(n_wg < cap ? n_wg : cap)), block(64 * wv);
  if (prologue == kProNone) {
    hipLaunchKernelGGL((decode_linear_kernel<C, MT, kProNone, EPI>), grid, block, 0, s, a);
  } else if (prologue == kProNorm) {
    hipLaunchKernelGGL((decode_linear_kernel<C, MT, kProNorm, EPI>), grid, block, 0, s, a);
  } else if constexpr (EPI == kEpiNone) {
    hipLaunchKernelGGL((decode_linear_kernel<C, MT, kProSwiglu, EPI>), grid, block, 0, s, a);
  }
}

template <int C, int MT> void launch_decode_linear_epi(DecodeLinearArgs a, int prologue, int epilogue, hipStream_t s) {
  constexpr int R = 8 / C;
  if (epilogue == kEpiNone) {
    a.n_groups = (a.N + R - 1) / R;
    launch_decode_linear_pro<C, MT, kEpiNone>(a, prologue, s);
    return;
  }
  if constexpr (R >= 2) {
    a.n_groups = (a.N / 2 + R / 2 - 1) / (R / 2);
    if (epilogue == kEpiSwiglu)
      launch_decode_linear_pro<C, MT, kEpiSwiglu>(a, prologue, s);
    else
      launch_decode_linear_pro<C, MT, kEpiConv>(a, prologue, s);
  }
}

template <int C> void launch_decode_linear(const DecodeLinearArgs& a, int prologue, int epilogue, hipStream_t s) {
  if constexpr (C == 8) {
    launch_decode_linear_epi<C, 4>(a, prologue, epilogue, s);  // 4096-wide rows: four activation rows fit the registers
  } else {
    if (a.M <= 4)
      launch_decode_linear_epi<C, 4>(a, prologue, epilogue, s);
    else
      launch_decode_linear_epi<C, 8>(a, prologue, epilogue, s);
  }
}

// whether the byte ranges [a, a + na) and [b, b + nb) intersect (an absent tensor intersects nothing)
static bool ranges_overlap(const void* a, int64_t na, const void* b, int64_t nb) {
  if (a == nullptr || b == nullptr || na <= 0 || nb <= 0) return false;
  const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
  return a0 < b0 + (uintptr_t)nb && b0 < a0 + (uintptr_t)na;
}

}  // namespace based

extern "C" BASED_API int based_decode_linear(const void* x, int64_t x_row_stride, const int64_t* x_row_index,
                                             int64_t x_index_rows, const void* weight, int64_t w_row_stride,
                                             const void* bias, void* y, int64_t y_row_stride, int64_t M,
                                             int64_t N, int64_t K, int prologue, const float* residual_in,
                                             int64_t ri_row_stride, float* residual_out, int64_t ro_row_stride,
                                             const void* norm_weight, float eps, int epilogue, void* conv_state,
                                             int conv_state_dtype, const void* conv_weight, const void* conv_bias,
                                             int conv_k, void* stream) {
  using namespace based;
  BASED_REQUIRE(x && weight && y, BASED_ERR_ARG, "decode_linear: null pointer argument");
  BASED_REQUIRE(M >= 0 && N > 0 && K > 0, BASED_ERR_ARG, "decode_linear: bad sizes");
  BASED_REQUIRE(M <= BASED_DECODE_LINEAR_MAX_ROWS, BASED_ERR_SHAPE,
                "decode_linear: %ld activation rows, at most %d (use a GEMM beyond that)", (long)M,
                BASED_DECODE_LINEAR_MAX_ROWS);
  BASED_REQUIRE(K % 8 == 0 && K <= 4096, BASED_ERR_SHAPE,
                "decode_linear: contraction length %ld unsupported (multiple of 8, at most 4096)", (long)K);
  BASED_REQUIRE(N < (1ll << 30), BASED_ERR_SHAPE, "decode_linear: too many output features");
  BASED_REQUIRE(prologue == kProNone || prologue == kProNorm || prologue == kProSwiglu, BASED_ERR_ARG,
                "decode_linear: unknown prologue %d", prologue);
  BASED_REQUIRE(epilogue == kEpiNone || epilogue == kEpiSwiglu || epilogue == kEpiConv, BASED_ERR_ARG,
                "decode_linear: unknown epilogue %d", epilogue);
  BASED_REQUIRE(x_row_stride % 8 == 0 && w_row_stride % 8 == 0, BASED_ERR_ALIGN,
                "decode_linear: row strides of x and weight must be multiples of 8 elements");
  uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight);
  if (prologue == kProNorm) {
    BASED_REQUIRE(norm_weight != nullptr, BASED_ERR_ARG, "decode_linear: the norm prologue needs its weight");
    BASED_REQUIRE(ri_row_stride % 4 == 0 && ro_row_stride % 4 == 0, BASED_ERR_ALIGN,
                  "decode_linear: residual row strides must be multiples of 4 elements");
    bits |= reinterpret_cast<uintptr_t>(residual_in) | reinterpret_cast<uintptr_t>(residual_out) |
            reinterpret_cast<uintptr_t>(norm_weight);
  } else {
    BASED_REQUIRE(residual_in == nullptr && residual_out == nullptr && norm_weight == nullptr, BASED_ERR_ARG,
                  "decode_linear: residual and norm arguments belong to the norm prologue");
  }
  if (epilogue != kEpiNone) {
    BASED_REQUIRE(N % 2 == 0, BASED_ERR_SHAPE, "decode_linear: a paired epilogue needs an even number of weight rows");
    BASED_REQUIRE(K <= 2048, BASED_ERR_SHAPE,
                  "decode_linear: paired epilogues take contraction lengths up to 2048 (got %ld)", (long)K);
    BASED_REQUIRE(prologue != kProSwiglu, BASED_ERR_ARG, "decode_linear: the gate prologue has no paired epilogue");
  }
  if (epilogue == kEpiConv) {
    BASED_REQUIRE(conv_state && conv_weight, BASED_ERR_ARG, "decode_linear: the convolution epilogue needs state and weight");
    BASED_REQUIRE(conv_k >= 2 && conv_k <= 4, BASED_ERR_SHAPE, "decode_linear: convolution kernel size %d (2 to 4)", conv_k);
    BASED_REQUIRE(conv_state_dtype == BASED_BF16 || conv_state_dtype == BASED_F32, BASED_ERR_DTYPE,
                  "decode_linear: bad convolution state dtype");
  } else {
    BASED_REQUIRE(conv_state == nullptr && conv_weight == nullptr && conv_bias == nullptr, BASED_ERR_ARG,
                  "decode_linear: convolution arguments belong to the convolution epilogue");
  }
  BASED_REQUIRE(x_row_index == nullptr || x_index_rows > 0, BASED_ERR_ARG,
                "decode_linear: a row index needs the number of rows it may address");
  BASED_REQUIRE((bits & 15) == 0, BASED_ERR_ALIGN, "decode_linear: tensors must be 16-byte aligned");
  if (M == 0) return BASED_OK;
  {
    // Every workgroup re-reads x and residual_in while workgroup 0 writes residual_out and the tails
    // write y: an output that overlaps an input, even partly (a view shifted by some rows), would be
    // a race between workgroups.  Compared as byte ranges.
    const int64_t x_rows = x_row_index ? x_index_rows : M;
    const int64_t x_bytes = ((x_rows - 1) * x_row_stride + (prologue == kProSwiglu ? 2 * K : K)) * 2;
    const int64_t ri_bytes = ((M - 1) * ri_row_stride + K) * 4, ro_bytes = ((M - 1) * ro_row_stride + K) * 4;
    const int64_t y_bytes = ((M - 1) * y_row_stride + (epilogue == kEpiNone ? N : N / 2)) * 2;
    BASED_REQUIRE(!ranges_overlap(residual_out, ro_bytes, residual_in, ri_bytes) &&
                      !ranges_overlap(residual_out, ro_bytes, x, x_bytes) && !ranges_overlap(y, y_bytes, x, x_bytes) &&
                      !ranges_overlap(y, y_bytes, residual_in, ri_bytes) && !ranges_overlap(y, y_bytes, residual_out, ro_bytes),
                  BASED_ERR_ARG, "decode_linear: an output (y, residual_out) overlaps an input or the other output");
  }

  DecodeLinearArgs a;
  a.x_sr = x_row_stride;
  a.x_index_rows = x_index_rows;
  a.w = static_cast<const __bf16*>(weight);
  a.w_sr = w_row_stride;
  a.bias = static_cast<const __bf16*>(bias);
  a.y_sr = y_row_stride;
  a.N = (int)N;
  a.K = (int)K;
  a.ri_sr = ri_row_stride;
  a.ro_sr = ro_row_stride;
  a.norm_w = static_cast<const __bf16*>(norm_weight);
  a.eps = eps;
  a.n_groups = 0;
  a.conv_state = conv_state;
  a.conv_w = static_cast<const __bf16*>(conv_weight);
  a.conv_b = static_cast<const __bf16*>(conv_bias);
  a.conv_k = conv_k;
  a.conv_state_f32 = conv_state_dtype == BASED_F32;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (int)((K + 511) / 512);
  a.M = (int)M;
  a.m0 = 0;
  a.x = static_cast<const __bf16*>(x);
  a.x_index = x_row_index;
  a.y = static_cast<__bf16*>(y);
  a.res_in = residual_in;
  a.res_out = residual_out;
  if (chunks <= 1)
    launch_decode_linear<1>(a, prologue, epilogue, s);
  else if (chunks <= 2)
    launch_decode_linear<2>(a, prologue, epilogue, s);
  else if (chunks <= 4)
    launch_decode_linear<4>(a, prologue, epilogue, s);
  else
    launch_decode_linear<8>(a, prologue, epilogue, s);
  return check_launch("decode_linear");
}
