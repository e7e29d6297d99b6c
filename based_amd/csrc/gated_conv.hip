// Gated short convolution of the Based stack for gfx950 (memory-bound, element-wise):
//   y[b,l,c] = silu( sum_j w[c,j] * u1[b, l-K+1+j, c] (+ bias[c]) ) * u2[b,l,c]
// with u = [u1 | u2] the (B, L, 2D) output of the block's input projection
// (based/models/mixers/convolution.py:195-210: depthwise causal Conv1d, SiLU, gate), plus the
// single-token form on a rolling (B, D, K) state (convolution.py:88-109).
// `gated` = 0 gives the convolution on its own, y = conv(u) (+ bias), u of width D: the
// ShortConvolution module used as a mixer by itself (convolution.py:47-87, the path without the
// fused CUDA kernel, which applies no activation).
//
// Prefill: a thread owns 16 bytes of channels (8 bf16 / 4 fp32) and walks kTokens consecutive
// tokens with the last K-1 inputs kept in registers, so every u element is read once (plus a
// K-1 row halo per token block) and every y element written once, all as 16-byte accesses that
// a wavefront coalesces into full rows.
#include "common.hpp"

namespace based {

constexpr int kConvTokens = 8;   // tokens per thread in the prefill kernel
constexpr int kConvMaxK = 4;      // supported kernel sizes: 2..4

template <typename T> struct Vec16;
template <> struct Vec16<__bf16> {
  static constexpr int kN = 8;
  typedef bf16x8 type;
};
template <> struct Vec16<float> {
  static constexpr int kN = 4;
  typedef f32x4 type;
};

__device__ __forceinline__ float silu(float a) { return a / (1.0f + __expf(-a)); }

template <typename T> __device__ __forceinline__ float load_as_f32(const void* p, long i) {
  return to_f32(reinterpret_cast<const T*>(p)[i]);
}
__device__ __forceinline__ float load_dyn(const void* p, long i, int dtype) {
  return dtype == BASED_BF16 ? load_as_f32<__bf16>(p, i) : load_as_f32<float>(p, i);
}
__device__ __forceinline__ void store_dyn(void* p, long i, int dtype, float x) {
  if (dtype == BASED_BF16)
    reinterpret_cast<__bf16*>(p)[i] = (__bf16)x;
  else
    reinterpret_cast<float*>(p)[i] = x;
}

template <typename T, int K>
__global__ __launch_bounds__(256) void gated_conv_prefill_kernel(
    const T* __restrict__ u, const T* __restrict__ weight, const T* __restrict__ bias, T* __restrict__ y,
    void* __restrict__ state, int L, int D, long u_sb, long u_sl, long y_sb, long y_sl, int state_dtype, int gated) {
  constexpr int N = Vec16<T>::kN;
  typedef typename Vec16<T>::type vec_t;
  const int c0 = (blockIdx.x * 256 + threadIdx.x) * N;  // first channel of this thread
  if (c0 >= D) return;
  const int l0 = blockIdx.y * kConvTokens;
  const int b = blockIdx.z;
  const T* u1 = u + b * u_sb + c0;
  const T* u2 = u1 + D;
  T* yo = y + b * y_sb + c0;

  // No load below sits under a condition, and no loaded value goes through a select: a load in
  // a branch is waited for at the end of the branch, one memory round trip after the other.
  // Rows that do not exist are fetched from a valid row and cleared (as bits) or never used.
  typedef __attribute__((ext_vector_type(4))) uint32_t bits_t;
  auto keep_if = [](vec_t x, bool keep) -> vec_t {
    const uint32_t m = keep ? 0xffffffffu : 0u;
    return __builtin_bit_cast(vec_t, __builtin_bit_cast(bits_t, x) & bits_t{m, m, m, m});
  };

  // filter taps: N * K consecutive elements; bias: N (an absent bias reads the taps and is cleared)
  float w[N][K], bs[N];
  {
    const vec_t* wp = reinterpret_cast<const vec_t*>(weight + (long)c0 * K);
    vec_t wv[K];
#pragma unroll
    for (int j = 0; j < K; ++j) wv[j] = wp[j];
    const vec_t bv = keep_if(*reinterpret_cast<const vec_t*>(bias != nullptr ? bias + c0 : weight + (long)c0 * K),
                             bias != nullptr);
#pragma unroll
    for (int c = 0; c < N; ++c) {
#pragma unroll
      for (int j = 0; j < K; ++j) w[c][j] = to_f32(wv[(c * K + j) / N][(c * K + j) % N]);
      bs[c] = to_f32(bv[c]);
    }
  }

  // the K-1 inputs before the block (zeros before the sequence start)
  float win[K][N];
#pragma unroll
  for (int j = 0; j < K - 1; ++j) {
    const int l = l0 - (K - 1) + j;
    const vec_t x = keep_if(*reinterpret_cast<const vec_t*>(u1 + (long)(l >= 0 ? l : 0) * u_sl), l >= 0);
#pragma unroll
    for (int c = 0; c < N; ++c) win[j][c] = to_f32(x[c]);
  }

  const int ntok = L - l0 < kConvTokens ? L - l0 : kConvTokens;
  const T* gate_src = gated ? u2 : u1;  // without a gate the second operand is fetched and ignored
  constexpr int kBatch = 4;  // tokens whose loads are in flight together
#pragma unroll
  for (int t0 = 0; t0 < kConvTokens; t0 += kBatch) {
    vec_t x1[kBatch], x2[kBatch];
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      const long row = l0 + (t0 + i < ntok ? t0 + i : ntok - 1);  // past the end: the last token again, unused
      x1[i] = *reinterpret_cast<const vec_t*>(u1 + row * u_sl);
      x2[i] = *reinterpret_cast<const vec_t*>(gate_src + row * u_sl);
    }
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      if (t0 + i < ntok) {
        vec_t out;
#pragma unroll
        for (int c = 0; c < N; ++c) {
          win[K - 1][c] = to_f32(x1[i][c]);
          float acc = bs[c];
#pragma unroll
          for (int j = 0; j < K; ++j) acc = __builtin_fmaf(w[c][j], win[j][c], acc);
          out[c] = from_f32<T>(gated ? silu(acc) * to_f32(x2[i][c]) : acc);
#pragma unroll
          for (int j = 0; j < K - 1; ++j) win[j][c] = win[j + 1][c];
        }
        *reinterpret_cast<vec_t*>(yo + (long)(l0 + t0 + i) * y_sl) = out;
      }
    }
  }

  // rolling state for decoding: the last K inputs of every channel, oldest first
  if (state != nullptr && l0 + ntok == L) {
#pragma unroll
    for (int c = 0; c < N; ++c) {
      const long base = ((long)b * D + c0 + c) * K;
      // after the last token the window holds inputs L-K+1 .. L-1 in win[0..K-2]; input L-K is
      // gone from it, so re-read it (it exists only if L >= K)
      float oldest = 0.0f;
      if (L - K >= 0) oldest = to_f32(u1[(long)(L - K) * u_sl + c]);
      store_dyn(state, base, state_dtype, oldest);
#pragma unroll
      for (int j = 1; j < K; ++j) store_dyn(state, base + j, state_dtype, win[j - 1][c]);
    }
  }
}

// Loads / stores COUNT consecutive elements (a multiple of 16 bytes, 16-byte aligned) as floats.
template <typename E, int COUNT> __device__ __forceinline__ void load_run(const void* p, long first, float (&out)[COUNT]) {
  constexpr int kPer = 16 / (int)sizeof(E);
  static_assert(COUNT % kPer == 0, "run must be whole 16-byte pieces");
  typedef typename Vec16<E>::type vec_t;
  const vec_t* src = reinterpret_cast<const vec_t*>(reinterpret_cast<const E*>(p) + first);
#pragma unroll
  for (int i = 0; i < COUNT / kPer; ++i) {
    const vec_t x = src[i];
#pragma unroll
    for (int j = 0; j < kPer; ++j) out[i * kPer + j] = to_f32(x[j]);
  }
}
template <typename E, int COUNT> __device__ __forceinline__ void store_run(void* p, long first, const float (&in)[COUNT]) {
  constexpr int kPer = 16 / (int)sizeof(E);
  typedef typename Vec16<E>::type vec_t;
  vec_t* dst = reinterpret_cast<vec_t*>(reinterpret_cast<E*>(p) + first);
#pragma unroll
  for (int i = 0; i < COUNT / kPer; ++i) {
    vec_t x;
#pragma unroll
    for (int j = 0; j < kPer; ++j) x[j] = from_f32<E>(in[i * kPer + j]);
    dst[i] = x;
  }
}

// A thread owns 8 consecutive channels: their K-entry state rows and weight rows are 8 K
// consecutive elements each, moved as 16-byte pieces.
template <typename T, typename TS, int K>
__global__ __launch_bounds__(256) void gated_conv_step_kernel(
    const T* __restrict__ u, TS* __restrict__ state, const T* __restrict__ weight, const T* __restrict__ bias,
    T* __restrict__ y, int B, int D, long u_sb, long y_sb, int gated) {
  constexpr int N = 8;
  const long item = (long)blockIdx.x * 256 + threadIdx.x;
  const int per_row = D / N;
  if (item >= (long)B * per_row) return;
  const int b = (int)(item / per_row);
  const int c0 = (int)(item % per_row) * N;
  float x1[N], x2[N] = {}, st[N * K], w[N * K], bs[N], out[N];
  load_run<T, N>(u + b * u_sb, c0, x1);
  if (gated) load_run<T, N>(u + b * u_sb, D + c0, x2);
  load_run<TS, N * K>(state, ((long)b * D + c0) * K, st);
  load_run<T, N * K>(weight, (long)c0 * K, w);
#pragma unroll
  for (int c = 0; c < N; ++c) bs[c] = 0.0f;
  if (bias != nullptr) load_run<T, N>(bias, c0, bs);
#pragma unroll
  for (int c = 0; c < N; ++c) {
#pragma unroll
    for (int j = 0; j < K - 1; ++j) st[c * K + j] = st[c * K + j + 1];  // roll by one
    st[c * K + K - 1] = x1[c];
    float acc = bs[c];
#pragma unroll
    for (int j = 0; j < K; ++j) acc = __builtin_fmaf(w[c * K + j], st[c * K + j], acc);
    out[c] = gated ? silu(acc) * x2[c] : acc;
  }
  store_run<TS, N * K>(state, ((long)b * D + c0) * K, st);
  store_run<T, N>(y + b * y_sb, c0, out);
}

// SwiGLU gate of the MLP: out = u[:, :F] * silu(u[:, F:]) (based/models/mlp.py:147-151).
template <typename T>
__global__ __launch_bounds__(256) void swiglu_kernel(const T* __restrict__ u, T* __restrict__ out, long rows, int F,
                                                     long u_sr, long o_sr) {
  constexpr int N = Vec16<T>::kN;
  typedef typename Vec16<T>::type vec_t;
  const long item = (long)blockIdx.x * 256 + threadIdx.x;
  const int per_row = F / N;
  if (item >= rows * per_row) return;
  const long r = item / per_row;
  const int c0 = (int)(item % per_row) * N;
  const vec_t a = *reinterpret_cast<const vec_t*>(u + r * u_sr + c0);
  const vec_t g = *reinterpret_cast<const vec_t*>(u + r * u_sr + F + c0);
  vec_t o;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    // torch rounds silu(gate) to the tensor dtype before the product
    const float sg = to_f32(from_f32<T>(silu(to_f32(g[i]))));
    o[i] = from_f32<T>(to_f32(a[i]) * sg);
  }
  *reinterpret_cast<vec_t*>(out + r * o_sr + c0) = o;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename T>
int launch_gated_conv_prefill(const void* u, const void* weight, const void* bias, void* y, void* state,
                              int64_t B, int64_t L, int64_t D, int K, int64_t u_sb, int64_t u_sl,
                              int64_t y_sb, int64_t y_sl, int state_dtype, int gated, hipStream_t stream) {
  constexpr int N = Vec16<T>::kN;
  dim3 grid((unsigned)((D / N + 255) / 256), (unsigned)((L + kConvTokens - 1) / kConvTokens), (unsigned)B), block(256);
#define BASED_CONV_CASE(KK)                                                                               \
  case KK:                                                                                                \
    hipLaunchKernelGGL((gated_conv_prefill_kernel<T, KK>), grid, block, 0, stream, (const T*)u,            \
                       (const T*)weight, (const T*)bias, (T*)y, state, (int)L, (int)D, u_sb, u_sl, y_sb,   \
                       y_sl, state_dtype, gated);                                                         \
    break;
  switch (K) {
    BASED_CONV_CASE(2)
    BASED_CONV_CASE(3)
    BASED_CONV_CASE(4)
  }
#undef BASED_CONV_CASE
  return check_launch("gated_conv_prefill");
}

template <typename T, typename TS>
int launch_gated_conv_step(const void* u, void* state, const void* weight, const void* bias, void* y,
                           int64_t B, int64_t D, int K, int64_t u_sb, int64_t y_sb, int gated, hipStream_t stream) {
  const int64_t items = B * (D / 8);
  dim3 grid((unsigned)((items + 255) / 256)), block(256);
#define BASED_CONV_CASE(KK)                                                                              \
  case KK:                                                                                               \
    hipLaunchKernelGGL((gated_conv_step_kernel<T, TS, KK>), grid, block, 0, stream, (const T*)u, (TS*)state, \
                       (const T*)weight, (const T*)bias, (T*)y, (int)B, (int)D, u_sb, y_sb, gated);       \
    break;
  switch (K) {
    BASED_CONV_CASE(2)
    BASED_CONV_CASE(3)
    BASED_CONV_CASE(4)
  }
#undef BASED_CONV_CASE
  return check_launch("gated_conv_step");
}

}  // namespace based

namespace based {
static int conv_prefill_impl(const char* who, int gated, const void* u, const void* weight, const void* bias, void* y,
                             void* state, int64_t B, int64_t L, int64_t D, int K, int64_t u_sb, int64_t u_sl,
                             int64_t y_sb, int64_t y_sl, int io_dtype, int state_dtype, void* stream) {
  BASED_REQUIRE(u && weight && y, BASED_ERR_ARG, "%s: null pointer argument", who);
  BASED_REQUIRE(B >= 0 && L >= 0 && D > 0, BASED_ERR_ARG, "%s: bad sizes", who);
  BASED_REQUIRE(io_dtype == BASED_BF16 || io_dtype == BASED_F32, BASED_ERR_DTYPE, "%s: bad io dtype", who);
  BASED_REQUIRE(state == nullptr || state_dtype == BASED_BF16 || state_dtype == BASED_F32, BASED_ERR_DTYPE,
                "%s: bad state dtype", who);
  BASED_REQUIRE(K >= 2 && K <= kConvMaxK, BASED_ERR_SHAPE, "%s: kernel size %d unsupported (2..4)", who, K);
  const int n = io_dtype == BASED_BF16 ? 8 : 4;
  BASED_REQUIRE(D % n == 0, BASED_ERR_SHAPE, "%s: channel count must be a multiple of %d", who, n);
  BASED_REQUIRE(u_sb % n == 0 && u_sl % n == 0 && y_sb % n == 0 && y_sl % n == 0, BASED_ERR_ALIGN,
                "%s: strides must be multiples of %d elements", who, n);
  BASED_REQUIRE(aligned16(u) && aligned16(y) && aligned16(weight) && aligned16(bias), BASED_ERR_ALIGN,
                "%s: tensors must be 16-byte aligned", who);
  BASED_REQUIRE(B < 65536 && (L + kConvTokens - 1) / kConvTokens < 65536, BASED_ERR_SHAPE,
                "%s: grid too large", who);
  if (B == 0 || L == 0) return BASED_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return io_dtype == BASED_BF16
             ? launch_gated_conv_prefill<__bf16>(u, weight, bias, y, state, B, L, D, K, u_sb, u_sl, y_sb, y_sl, state_dtype, gated, s)
             : launch_gated_conv_prefill<float>(u, weight, bias, y, state, B, L, D, K, u_sb, u_sl, y_sb, y_sl, state_dtype, gated, s);
}
}  // namespace based

namespace based {
static int conv_step_impl(const char* who, int gated, const void* u, void* state, const void* weight, const void* bias,
                          void* y, int64_t B, int64_t D, int K, int64_t u_sb, int64_t y_sb, int io_dtype,
                          int state_dtype, void* stream) {
  BASED_REQUIRE(u && state && weight && y, BASED_ERR_ARG, "%s: null pointer argument", who);
  BASED_REQUIRE(B >= 0 && D > 0, BASED_ERR_ARG, "%s: bad sizes", who);
  BASED_REQUIRE(io_dtype == BASED_BF16 || io_dtype == BASED_F32, BASED_ERR_DTYPE, "%s: bad io dtype", who);
  BASED_REQUIRE(state_dtype == BASED_BF16 || state_dtype == BASED_F32, BASED_ERR_DTYPE, "%s: bad state dtype", who);
  BASED_REQUIRE(K >= 2 && K <= kConvMaxK, BASED_ERR_SHAPE, "%s: kernel size %d unsupported (2..4)", who, K);
  BASED_REQUIRE(D % 8 == 0, BASED_ERR_SHAPE, "%s: channel count must be a multiple of 8", who);
  BASED_REQUIRE(u_sb % 8 == 0 && y_sb % 8 == 0, BASED_ERR_ALIGN, "%s: strides must be multiples of 8 elements", who);
  BASED_REQUIRE(aligned16(u) && aligned16(y) && aligned16(state) && aligned16(weight) && aligned16(bias),
                BASED_ERR_ALIGN, "%s: tensors must be 16-byte aligned", who);
  BASED_REQUIRE(B * (D / 8) < (1ll << 39), BASED_ERR_SHAPE, "%s: grid too large", who);
  if (B == 0) return BASED_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (io_dtype == BASED_BF16)
    return state_dtype == BASED_BF16 ? launch_gated_conv_step<__bf16, __bf16>(u, state, weight, bias, y, B, D, K, u_sb, y_sb, gated, s)
                                     : launch_gated_conv_step<__bf16, float>(u, state, weight, bias, y, B, D, K, u_sb, y_sb, gated, s);
  return state_dtype == BASED_BF16 ? launch_gated_conv_step<float, __bf16>(u, state, weight, bias, y, B, D, K, u_sb, y_sb, gated, s)
                                   : launch_gated_conv_step<float, float>(u, state, weight, bias, y, B, D, K, u_sb, y_sb, gated, s);
}
}  // namespace based

extern "C" BASED_API int based_gated_conv_prefill(const void* u, const void* weight, const void* bias, void* y,
                                                  void* state, int64_t B, int64_t L, int64_t D, int K,
                                                  int64_t u_sb, int64_t u_sl, int64_t y_sb, int64_t y_sl,
                                                  int io_dtype, int state_dtype, void* stream) {
  return based::conv_prefill_impl("gated_conv_prefill", 1, u, weight, bias, y, state, B, L, D, K, u_sb, u_sl, y_sb, y_sl,
                                  io_dtype, state_dtype, stream);
}

extern "C" BASED_API int based_gated_conv_step(const void* u, void* state, const void* weight, const void* bias,
                                               void* y, int64_t B, int64_t D, int K, int64_t u_sb, int64_t y_sb,
                                               int io_dtype, int state_dtype, void* stream) {
  return based::conv_step_impl("gated_conv_step", 1, u, state, weight, bias, y, B, D, K, u_sb, y_sb, io_dtype,
                               state_dtype, stream);
}

extern "C" BASED_API int based_short_conv_prefill(const void* u, const void* weight, const void* bias, void* y,
                                                  void* state, int64_t B, int64_t L, int64_t D, int K,
                                                  int64_t u_sb, int64_t u_sl, int64_t y_sb, int64_t y_sl,
                                                  int io_dtype, int state_dtype, void* stream) {
  return based::conv_prefill_impl("short_conv_prefill", 0, u, weight, bias, y, state, B, L, D, K, u_sb, u_sl, y_sb, y_sl,
                                  io_dtype, state_dtype, stream);
}

extern "C" BASED_API int based_short_conv_step(const void* u, void* state, const void* weight, const void* bias,
                                               void* y, int64_t B, int64_t D, int K, int64_t u_sb, int64_t y_sb,
                                               int io_dtype, int state_dtype, void* stream) {
  return based::conv_step_impl("short_conv_step", 0, u, state, weight, bias, y, B, D, K, u_sb, y_sb, io_dtype,
                               state_dtype, stream);
}

extern "C" BASED_API int based_swiglu(const void* u, void* out, int64_t rows, int64_t F, int64_t u_sr, int64_t o_sr,
                                      int io_dtype, void* stream) {
  using namespace based;
  BASED_REQUIRE(u && out, BASED_ERR_ARG, "swiglu: null pointer argument");
  BASED_REQUIRE(rows >= 0 && F > 0, BASED_ERR_ARG, "swiglu: bad sizes");
  BASED_REQUIRE(io_dtype == BASED_BF16 || io_dtype == BASED_F32, BASED_ERR_DTYPE, "swiglu: bad dtype");
  const int n = io_dtype == BASED_BF16 ? 8 : 4;
  BASED_REQUIRE(F % n == 0, BASED_ERR_SHAPE, "swiglu: width must be a multiple of %d", n);
  BASED_REQUIRE(u_sr % n == 0 && o_sr % n == 0, BASED_ERR_ALIGN, "swiglu: strides must be multiples of %d elements", n);
  BASED_REQUIRE(aligned16(u) && aligned16(out), BASED_ERR_ALIGN, "swiglu: tensors must be 16-byte aligned");
  const int64_t items = rows * (F / n);
  BASED_REQUIRE((items + 255) / 256 < (1ll << 31), BASED_ERR_SHAPE, "swiglu: grid too large");
  if (rows == 0) return BASED_OK;
  dim3 grid((unsigned)((items + 255) / 256)), block(256);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (io_dtype == BASED_BF16)
    hipLaunchKernelGGL(swiglu_kernel<__bf16>, grid, block, 0, s, (const __bf16*)u, (__bf16*)out, (long)rows, (int)F, u_sr, o_sr);
  else
    hipLaunchKernelGGL(swiglu_kernel<float>, grid, block, 0, s, (const float*)u, (float*)out, (long)rows, (int)F, u_sr, o_sr);
  return check_launch("swiglu");
}
