// Greedy sampling of one decoding step, with the bookkeeping that the next step needs, for gfx950.
//
// After the LM head of a single-token step the reference's loop picks logits.argmax(-1)
// (based/generation.py:64-70, top_k == 1), appends it to the sequences, makes it the next input
// and advances seqlen_offset (generation.py:171-204): an argmax kernel, a concatenation, and in a
// loop that replays a recorded graph three more small copies and fills per token.  Here all of it
// is ONE launch that can be recorded in the same graph as the step itself: per batch row, one
// workgroup finds the first index of the largest logit (NaN counts as the largest, as in torch)
// and writes the token to the next step's input buffer and to the row of generated sequences at
// the position after the one just processed, then advances the device-side position counters
// the step kernels read.
#include "common.hpp"

namespace based {

// (value, index) candidates: a beats b when it is larger, or NaN against a number; equal
// candidates keep the lower index
__device__ __forceinline__ bool greedy_beats(float va, int ia, float vb, int ib) {
  const bool a_nan = va != va, b_nan = vb != vb;
  if (a_nan || b_nan) return a_nan && (!b_nan || ia < ib);
  return va > vb || (va == vb && ia < ib);
}

constexpr int kGreedyThreads = 1024;

template <typename T>
__global__ __launch_bounds__(kGreedyThreads) void greedy_step_kernel(
    const T* __restrict__ logits, long logits_stride, int V, int64_t* __restrict__ next_ids, long ids_stride,
    int64_t* __restrict__ sequences, long seq_stride, int seq_len, int32_t* __restrict__ lengths,
    int64_t* __restrict__ position_ids, long pos_stride, int vec_ok) {
  __shared__ float s_val[kGreedyThreads / kWave];
  __shared__ int s_idx[kGreedyThreads / kWave];
  const int b = blockIdx.x;
  const int tid = threadIdx.x;
  const T* row = logits + (long)b * logits_stride;
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  constexpr int kVec = 16 / (int)sizeof(T);  // elements per 16-byte load
  int done = 0;
  if (vec_ok) {
    const int n_vec = V / kVec;
    for (int j = tid; j < n_vec; j += kGreedyThreads) {
      if constexpr (sizeof(T) == 2) {
        const bf16x8 x = *reinterpret_cast<const bf16x8*>(row + (long)j * kVec);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const float v = to_f32(x[e]);
          if (greedy_beats(v, j * kVec + e, best, best_i)) best = v, best_i = j * kVec + e;
        }
      } else {
        const f32x4 x = *reinterpret_cast<const f32x4*>(row + (long)j * kVec);
#pragma unroll
        for (int e = 0; e < kVec; ++e)
          if (greedy_beats(x[e], j * kVec + e, best, best_i)) best = x[e], best_i = j * kVec + e;
      }
    }
    done = n_vec * kVec;
  }
  for (int i = done + tid; i < V; i += kGreedyThreads) {
    const float v = to_f32(row[i]);
    if (greedy_beats(v, i, best, best_i)) best = v, best_i = i;
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) {
    const float ov = __shfl_xor(best, m, 64);
    const int oi = __shfl_xor(best_i, m, 64);
    if (greedy_beats(ov, oi, best, best_i)) best = ov, best_i = oi;
  }
  if ((tid & 63) == 0) s_val[tid >> 6] = best, s_idx[tid >> 6] = best_i;
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < kGreedyThreads / kWave; ++w)
      if (greedy_beats(s_val[w], s_idx[w], best, best_i)) best = s_val[w], best_i = s_idx[w];
    const int64_t tok = best_i;
    const int p = lengths[b];  // position of the token this step processed
    next_ids[(long)b * ids_stride] = tok;
    if (sequences != nullptr && p + 1 >= 0 && p + 1 < seq_len) sequences[(long)b * seq_stride + p + 1] = tok;
    lengths[b] = p + 1;
    if (position_ids != nullptr) position_ids[(long)b * pos_stride] = p + 1;
  }
}

}  // namespace based

extern "C" BASED_API int based_greedy_step(const void* logits, int64_t B, int64_t V, int64_t logits_stride,
                                           int64_t* next_ids, int64_t ids_stride, int64_t* sequences,
                                           int64_t seq_stride, int64_t seq_len, int32_t* lengths,
                                           int64_t* position_ids, int64_t pos_stride, int io_dtype, void* stream) {
  using namespace based;
  BASED_REQUIRE(logits && next_ids && lengths, BASED_ERR_ARG, "greedy_step: null pointer argument");
  BASED_REQUIRE(B >= 0 && B < (1ll << 31) && V > 0 && V < (1ll << 31) && seq_len >= 0 && seq_len < (1ll << 31),
                BASED_ERR_ARG, "greedy_step: bad sizes B=%ld V=%ld seq_len=%ld", (long)B, (long)V, (long)seq_len);
  BASED_REQUIRE(logits_stride >= V, BASED_ERR_ARG, "greedy_step: logits row stride %ld below the vocabulary %ld",
                (long)logits_stride, (long)V);
  BASED_REQUIRE(io_dtype == BASED_BF16 || io_dtype == BASED_F32, BASED_ERR_DTYPE, "greedy_step: io_dtype %d unsupported",
                io_dtype);
  if (B == 0) return BASED_OK;
  const int elt = io_dtype == BASED_BF16 ? 2 : 4;
  const int vec_ok = (reinterpret_cast<uintptr_t>(logits) & 15) == 0 && (logits_stride * elt) % 16 == 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (io_dtype == BASED_BF16)
    hipLaunchKernelGGL(greedy_step_kernel<__bf16>, dim3((unsigned)B), dim3(kGreedyThreads), 0, s, (const __bf16*)logits,
                       logits_stride, (int)V, next_ids, ids_stride, sequences, seq_stride, (int)seq_len, lengths,
                       position_ids, pos_stride, vec_ok);
  else
    hipLaunchKernelGGL(greedy_step_kernel<float>, dim3((unsigned)B), dim3(kGreedyThreads), 0, s, (const float*)logits,
                       logits_stride, (int)V, next_ids, ids_stride, sequences, seq_stride, (int)seq_len, lengths,
                       position_ids, pos_stride, vec_ok);
  return check_launch("greedy_step");
}
