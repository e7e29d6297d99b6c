// Residual add + RMSNorm of the prenorm block for gfx950 (memory-bound, one pass):
//   r   = x + residual            (fp32; r = x for the first block)
//   y   = rms_norm(round(r)) * w  (round = cast to the dtype of x, as the block hands the norm
//                                  `residual.to(dtype=norm.weight.dtype)`: block.py:136-139,151-155)
//   out = r                       (kept in fp32 when residual_in_fp32)
// with rms_norm(v) = v * rsqrt(mean(v^2) + eps) evaluated in fp32
// (based/ops/triton/layer_norm.py:117-118).  In plain torch this is about ten element-wise and
// reduction launches per norm; here one wavefront owns a row and touches every element once.
#include "common.hpp"

namespace based {

// (not const: constant data lives in another address space, and a pointer that may be in either
// makes the load a flat one, which is waited for on the spot)
__device__ __attribute__((aligned(32))) uint32_t kNormZeroPage[8] = {};

constexpr int kNormMaxChunks = 8;  // a lane holds up to 8 chunks of 8 elements: rows up to 4096 wide

template <typename T> __device__ __forceinline__ void load8(const T* p, float (&v)[8]);
template <> __device__ __forceinline__ void load8<__bf16>(const __bf16* p, float (&v)[8]) {
  const bf16x8 x = *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = to_f32(x[i]);
}
template <> __device__ __forceinline__ void load8<float>(const float* p, float (&v)[8]) {
  const f32x4 a = reinterpret_cast<const f32x4*>(p)[0], b = reinterpret_cast<const f32x4*>(p)[1];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[i] = a[i];
    v[4 + i] = b[i];
  }
}
template <typename T> __device__ __forceinline__ void store8(T* p, const float (&v)[8]);
template <> __device__ __forceinline__ void store8<__bf16>(__bf16* p, const float (&v)[8]) {
  typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
  const u32x4 w = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7])};
  *reinterpret_cast<u32x4*>(p) = w;
}
template <> __device__ __forceinline__ void store8<float>(float* p, const float (&v)[8]) {
  reinterpret_cast<f32x4*>(p)[0] = f32x4{v[0], v[1], v[2], v[3]};
  reinterpret_cast<f32x4*>(p)[1] = f32x4{v[4], v[5], v[6], v[7]};
}

// TX: dtype of x, y and the weight; TR: dtype of the residual stream (in and out).
template <typename TX, typename TR, int NCH>
__global__ __launch_bounds__(256) void add_rms_norm_kernel(
    const TX* __restrict__ x, const TR* __restrict__ res_in, const TX* __restrict__ weight, TX* __restrict__ y,
    TR* __restrict__ res_out, long rows, int D, long x_sr, long ri_sr, long y_sr, long ro_sr, float eps) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  x += row * x_sr;
  y += row * y_sr;
  if (res_in != nullptr) res_in += row * ri_sr;
  if (res_out != nullptr) res_out += row * ro_sr;

  // Every load is issued unconditionally and up front (a load under a condition is waited for at
  // the end of its branch, one round trip after the other): chunks past the row end re-read the
  // start of the row (and are not used), an absent residual reads a page of zeros.
  float v[NCH][8], w[NCH][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e0 = (c * 64 + lane) * 8;
    const int ec = e0 < D ? e0 : 0;
    load8<TX>(x + ec, v[c]);
    load8<TX>(weight + ec, w[c]);
    float r[8];
    load8<TR>(res_in != nullptr ? res_in + ec : reinterpret_cast<const TR*>(kNormZeroPage), r);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[c][i] += r[i];
  }
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e0 = (c * 64 + lane) * 8;
    if (e0 < D) {
      if (res_out != nullptr) store8<TR>(res_out + e0, v[c]);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        v[c][i] = to_f32(from_f32<TX>(v[c][i]));  // the norm sees the sum in the dtype of x
        ss = __builtin_fmaf(v[c][i], v[c][i], ss);
      }
    }
  }
  ss = wave_sum(ss);
  const float rstd = rsqrtf(ss / (float)D + eps);
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e0 = (c * 64 + lane) * 8;
    if (e0 < D) {
      float o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = v[c][i] * rstd * w[c][i];
      store8<TX>(y + e0, o);
    }
  }
}

template <typename TX, typename TR>
int launch_add_rms_norm(const void* x, const void* res_in, const void* weight, void* y, void* res_out,
                        int64_t rows, int64_t D, int64_t x_sr, int64_t ri_sr, int64_t y_sr, int64_t ro_sr,
                        float eps, hipStream_t stream) {
  dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  const int chunks = (int)((D + 511) / 512);
#define BASED_NORM_CASE(N)                                                                                   \
  hipLaunchKernelGGL((add_rms_norm_kernel<TX, TR, N>), grid, block, 0, stream, (const TX*)x, (const TR*)res_in, \
                     (const TX*)weight, (TX*)y, (TR*)res_out, (long)rows, (int)D, x_sr, ri_sr, y_sr, ro_sr, eps)
  if (chunks <= 1) {
    BASED_NORM_CASE(1);
  } else if (chunks <= 2) {
    BASED_NORM_CASE(2);
  } else if (chunks <= 4) {
    BASED_NORM_CASE(4);
  } else {
    BASED_NORM_CASE(8);
  }
#undef BASED_NORM_CASE
  return check_launch("add_rms_norm");
}

}  // namespace based

extern "C" BASED_API int based_add_rms_norm(const void* x, const void* residual_in, const void* weight, void* y,
                                            void* residual_out, int64_t rows, int64_t D, int64_t x_sr,
                                            int64_t ri_sr, int64_t y_sr, int64_t ro_sr, float eps, int x_dtype,
                                            int residual_dtype, void* stream) {
  using namespace based;
  BASED_REQUIRE(x && weight && y, BASED_ERR_ARG, "add_rms_norm: null pointer argument");
  BASED_REQUIRE(rows >= 0 && D > 0, BASED_ERR_ARG, "add_rms_norm: bad sizes");
  BASED_REQUIRE(x_dtype == BASED_BF16 || x_dtype == BASED_F32, BASED_ERR_DTYPE, "add_rms_norm: bad x dtype");
  BASED_REQUIRE(residual_dtype == BASED_BF16 || residual_dtype == BASED_F32, BASED_ERR_DTYPE,
                "add_rms_norm: bad residual dtype");
  BASED_REQUIRE(D % 8 == 0 && D <= 512 * kNormMaxChunks, BASED_ERR_SHAPE,
                "add_rms_norm: row width %ld unsupported (multiple of 8, at most %d)", (long)D, 512 * kNormMaxChunks);
  BASED_REQUIRE(x_sr % 8 == 0 && ri_sr % 8 == 0 && y_sr % 8 == 0 && ro_sr % 8 == 0, BASED_ERR_ALIGN,
                "add_rms_norm: row strides must be multiples of 8 elements");
  const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(residual_in) |
                         reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(y) |
                         reinterpret_cast<uintptr_t>(residual_out);
  BASED_REQUIRE((bits & 15) == 0, BASED_ERR_ALIGN, "add_rms_norm: tensors must be 16-byte aligned");
  BASED_REQUIRE((rows + 3) / 4 < (1ll << 31), BASED_ERR_SHAPE, "add_rms_norm: too many rows");
  if (rows == 0) return BASED_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (x_dtype == BASED_BF16)
    return residual_dtype == BASED_F32
               ? launch_add_rms_norm<__bf16, float>(x, residual_in, weight, y, residual_out, rows, D, x_sr, ri_sr, y_sr, ro_sr, eps, s)
               : launch_add_rms_norm<__bf16, __bf16>(x, residual_in, weight, y, residual_out, rows, D, x_sr, ri_sr, y_sr, ro_sr, eps, s);
  BASED_REQUIRE(residual_dtype == BASED_F32, BASED_ERR_DTYPE, "add_rms_norm: fp32 x needs an fp32 residual");
  return launch_add_rms_norm<float, float>(x, residual_in, weight, y, residual_out, rows, D, x_sr, ri_sr, y_sr, ro_sr, eps, s);
}
