// Measurement probes of bench.py (a library of their own, libbench_probes.so; not part of the
// product library and not declared in its header): plain streaming kernels with the memory access
// patterns of the hot kernels and no arithmetic to speak of.  What they reach on a given machine is the ceiling the real
// kernels are measured against next to the published HBM figure (the benchmark reports both).
//   stream_qkv : reads a packed (B, L, 3, H, 64) bf16 tensor and writes a (B, L, H, 64) one the way
//                the window-attention prefill does: a workgroup walks a run of tokens of G
//                neighbouring heads, every load instruction covering whole 128 G-byte pieces.
//   rmw        : reads and rewrites a float buffer in 16-byte pieces, lane-contiguous, like the
//                state update of the recurrent decode step.
//   copy       : plain 16-byte-per-lane copy of known size; the calibration kernel for the
//                profiler's HBM byte counters.
//   stream_prefill : the q / k / v reads and y writes of the chunked linear-attention prefill, chunk
//                by chunk per (batch, head), with no arithmetic: the memory ceiling of that kernel.
//   mfma       : nothing but independent dense bf16 MFMA 16x16x32 on non-zero register operands,
//                four workgroups of four wavefronts per compute unit: the rate the matrix pipes
//                sustain at the clock the board holds under that load (the published peak assumes
//                the maximum clock).
//
//   timestamp  : one lane stores the constant-rate device clock (wall_clock64).  Recorded in a graph in
//                front of and behind a run of launches, two of them time exactly that run from
//                inside the stream, where HIP events cannot be recorded (a graph holds no timing
//                events on this platform) and events around a whole graph launch also count the
//                boundary between two graph launches.
//
// Every entry point returns 0, or 1 for arguments it does not take.
#include <hip/hip_runtime.h>
#include <stdint.h>

#define PROBE_API extern "C" __attribute__((visibility("default")))
#define PROBE_REQUIRE(cond) \
  do {                      \
    if (!(cond)) return 1;  \
  } while (0)

namespace bench_probes {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

template <int G>
__global__ __launch_bounds__(256) void probe_stream_qkv_kernel(const u32x4* __restrict__ x, u32x4* __restrict__ o,
                                                               int B, int H, int L, int runs) {
  // 16-byte pieces: a token row of x holds 3*H*8 of them, one of o H*8
  const int t = threadIdx.x;
  const int groups = H / G;
  int id = blockIdx.x;
  const int run = id % runs;
  id /= runs;
  const int hg = id % groups, b = id / groups;
  if (b >= B) return;
  constexpr int kTokPerIter = 64 / G;   // 64 rows of 128 bytes per tensor and iteration, as one attention tile
  const int toks = (L + runs - 1) / runs;
  for (int t0 = run * toks; t0 < (run + 1) * toks && t0 < L; t0 += kTokPerIter) {
    u32x4 a[2][3];
    size_t oidx[2];
    bool live[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int p = t + 256 * i;
      const int tok = t0 + p / (8 * G), rem = p % (8 * G);
      const int head = hg * G + rem / 8, c = rem % 8;
      live[i] = tok < L && tok < (run + 1) * toks;
      oidx[i] = ((size_t)b * L + tok) * H * 8 + head * 8 + c;
#pragma unroll
      for (int s = 0; s < 3; ++s) {
        a[i][s] = u32x4{0, 0, 0, 0};
        if (live[i]) a[i][s] = x[(((size_t)b * L + tok) * 3 + s) * H * 8 + head * 8 + c];
      }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
      if (live[i]) __builtin_nontemporal_store(a[i][0] ^ a[i][1] ^ a[i][2], o + oidx[i]);
  }
}

template <bool WRITE>
__global__ __launch_bounds__(256) void probe_rw_kernel(u32x4* dst, const u32x4* src, size_t n16) {
  // grid-stride over 16-byte pieces, four in flight per lane
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += 4 * stride) {
    u32x4 a[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      a[u] = u32x4{0, 0, 0, 0};
      if (i + u * stride < n16) a[u] = __builtin_nontemporal_load(src + i + u * stride);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i + u * stride < n16) __builtin_nontemporal_store(WRITE ? a[u] : a[u] + u32x4{1, 1, 1, 1}, dst + i + u * stride);
  }
}

// stream_prefill: the memory side of the chunked linear-attention prefill with nothing else: one
// workgroup of 512 threads per (batch, head) walks the sequence in chunks of 64 tokens, fetching the
// chunk's q and k rows (32 bytes each), v rows (128 bytes) two chunks ahead and storing a y row
// (128 bytes) per token, in the (B, L, H*d) layout of the projections; 80,000 bytes of LDS are
// requested so that two workgroups share a compute unit as in the real kernel, and workgroup
// numbers are laid along the XCDs the same way.
__global__ __launch_bounds__(512, 4) void probe_stream_prefill_kernel(const u32x4* __restrict__ q, const u32x4* __restrict__ k,
                                                                       const u32x4* __restrict__ v, u32x4* __restrict__ y,
                                                                       int H, int L) {
  extern __shared__ unsigned char probe_lds[];
  const int t = threadIdx.x;
  const long n = gridDim.x;
  const long bh = (n % 8 == 0) ? (blockIdx.x % 8) * (n / 8) + blockIdx.x / 8 : blockIdx.x;
  const long b = bh / H, h = bh % H;
  // 16-byte pieces: a token row of q / k holds 2 H, of v / y 8 H
  const u32x4* qb = q + (b * L * H + h) * 2;
  const u32x4* kb = k + (b * L * H + h) * 2;
  const u32x4* vb = v + (b * L * H + h) * 8;
  u32x4* yb = y + (b * L * H + h) * 8;
  const int qrow = (t & 127) >> 1, qpc = t & 1;   // threads 0..127 fetch q, 128..255 k
  const int vrow = t >> 3, vpc = t & 7;
  const int chunks = L / 64;
  u32x4 a[3], c[3];
  auto fetch = [&](int ch, int slot) {
    const long tq = (long)ch * 64 + qrow, tv = (long)ch * 64 + vrow;
    a[slot] = t < 256 ? (t < 128 ? qb : kb)[tq * H * 2 + qpc] : u32x4{0, 0, 0, 0};   // 256 threads cover q and k
    c[slot] = vb[tv * H * 8 + vpc];
  };
  if (chunks > 0) fetch(0, 0);
  if (chunks > 1) fetch(1, 1);
  for (int ch = 0; ch < chunks; ch += 3) {
#pragma unroll
    for (int u = 0; u < 3; ++u) {
      if (ch + u < chunks) {
        if (ch + u + 2 < chunks) fetch(ch + u + 2, (u + 2) % 3);
        __builtin_nontemporal_store(a[u] ^ c[u], yb + ((long)(ch + u) * 64 + vrow) * H * 8 + vpc);
      }
    }
  }
  if (t == 0 && probe_lds[0] == 123 && L < 0) yb[0] = u32x4{0, 0, 0, 0};  // keeps the LDS request alive
}

static bool probe_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace bench_probes

namespace bench_probes {
typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8;
typedef __attribute__((ext_vector_type(4))) float probe_f32x4;
constexpr int kMfmaPerIter = 32;   // 4 rounds over 8 independent accumulators

__global__ __launch_bounds__(256) void probe_mfma_kernel(float* __restrict__ out, int iters) {
  probe_f32x4 m[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) m[i] = probe_f32x4{0.f, 0.f, 0.f, 0.f};
  probe_bf16x8 a, b;
  unsigned s = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    s = s * 1664525u + 1013904223u;
    a[i] = (__bf16)(((int)(s >> 16) % 2001 - 1000) * 1e-3f);
    s = s * 1664525u + 1013904223u;
    b[i] = (__bf16)(((int)(s >> 16) % 2001 - 1000) * 1e-3f);
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < kMfmaPerIter / 8; ++r)
#pragma unroll
      for (int i = 0; i < 8; ++i) m[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, m[i], 0, 0, 0);
  }
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) acc += m[i][0] + m[i][1] + m[i][2] + m[i][3];
  out[blockIdx.x * blockDim.x + threadIdx.x] = acc;
}
__global__ __launch_bounds__(64) void probe_timestamp_kernel(uint64_t* out) {
  if (threadIdx.x == 0) *out = wall_clock64();
}
}  // namespace bench_probes

// Stores the device's constant-rate clock at *out (device memory, 8-byte aligned) when the launch runs.
PROBE_API int bench_probe_timestamp(void* out, void* stream) {
  using namespace bench_probes;
  PROBE_REQUIRE(out && (reinterpret_cast<uintptr_t>(out) & 7) == 0);
  hipLaunchKernelGGL(probe_timestamp_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), (uint64_t*)out);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

// Rate of that clock in kHz (0 if the runtime cannot tell).
PROBE_API int64_t bench_probe_clock_khz() {
  int dev = 0, khz = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess) return 0;
  return khz;
}

// `out` takes workgroups * 256 floats; *flops (host) receives the floating-point operations of the launch.
PROBE_API int bench_probe_mfma(float* out, int64_t workgroups, int64_t iters, double* flops, void* stream) {
  using namespace bench_probes;
  PROBE_REQUIRE(out && flops && workgroups > 0 && workgroups < (1ll << 20) && iters > 0 && iters < (1ll << 24));
  *flops = (double)workgroups * 4.0 * (double)iters * kMfmaPerIter * (2.0 * 16 * 16 * 32);
  hipLaunchKernelGGL(probe_mfma_kernel, dim3((unsigned)workgroups), dim3(256), 0, static_cast<hipStream_t>(stream), out,
                     (int)iters);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

PROBE_API int bench_probe_stream_qkv(const void* qkv, void* o, int64_t B, int64_t H, int64_t L,
                                                int heads_per_group, void* stream) {
  using namespace bench_probes;
  PROBE_REQUIRE(qkv && o);
  PROBE_REQUIRE(B > 0 && H > 0 && L > 0 && B < 65536 && H < 65536 && L < (1ll << 30));
  PROBE_REQUIRE(heads_per_group == 1 || heads_per_group == 2 || heads_per_group == 4);
  PROBE_REQUIRE(H % heads_per_group == 0);
  PROBE_REQUIRE(probe_aligned16(qkv) && probe_aligned16(o));
  // as the attention launcher: runs long enough to leave about 1024 x 256 threads in flight
  const int64_t n_tiles = (L + 63) / 64;
  int64_t run_tiles = B * H * n_tiles / 1024;
  run_tiles = run_tiles < 1 ? 1 : (run_tiles > n_tiles ? n_tiles : run_tiles);
  const int64_t runs = (n_tiles + run_tiles - 1) / run_tiles * heads_per_group;
  const int64_t grid = B * (H / heads_per_group) * runs;
  PROBE_REQUIRE(grid < (1ll << 31));
  auto kern = heads_per_group == 1 ? probe_stream_qkv_kernel<1>
                                   : (heads_per_group == 2 ? probe_stream_qkv_kernel<2> : probe_stream_qkv_kernel<4>);
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                     (const u32x4*)qkv, (u32x4*)o, (int)B, (int)H, (int)L, (int)runs);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

PROBE_API int bench_probe_rmw(void* buf, int64_t bytes, void* stream) {
  using namespace bench_probes;
  PROBE_REQUIRE(buf && bytes > 0 && bytes % 16 == 0);
  PROBE_REQUIRE(probe_aligned16(buf));
  hipLaunchKernelGGL(probe_rw_kernel<false>, dim3(256 * 8), dim3(256), 0, static_cast<hipStream_t>(stream),
                     (u32x4*)buf, (const u32x4*)buf, (size_t)(bytes / 16));
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

PROBE_API int bench_probe_copy(void* dst, const void* src, int64_t bytes, void* stream) {
  using namespace bench_probes;
  PROBE_REQUIRE(dst && src && bytes > 0 && bytes % 16 == 0);
  PROBE_REQUIRE(probe_aligned16(dst) && probe_aligned16(src));
  hipLaunchKernelGGL(probe_rw_kernel<true>, dim3(256 * 8), dim3(256), 0, static_cast<hipStream_t>(stream),
                     (u32x4*)dst, (const u32x4*)src, (size_t)(bytes / 16));
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

PROBE_API int bench_probe_stream_prefill(const void* q, const void* k, const void* v, void* y, int64_t B, int64_t H,
                                         int64_t L, void* stream) {
  using namespace bench_probes;
  PROBE_REQUIRE(q && k && v && y && B > 0 && H > 0 && L > 0 && L % 64 == 0 && B * H < (1ll << 31) && L < (1ll << 30));
  PROBE_REQUIRE(probe_aligned16(q) && probe_aligned16(k) && probe_aligned16(v) && probe_aligned16(y));
  static bool allowed = false;
  if (!allowed) {
    PROBE_REQUIRE(hipFuncSetAttribute(reinterpret_cast<const void*>(probe_stream_prefill_kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 80000) == hipSuccess);
    allowed = true;
  }
  hipLaunchKernelGGL(probe_stream_prefill_kernel, dim3((unsigned)(B * H)), dim3(512), 80000, static_cast<hipStream_t>(stream),
                     (const u32x4*)q, (const u32x4*)k, (const u32x4*)v, (u32x4*)y, (int)H, (int)L);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}
