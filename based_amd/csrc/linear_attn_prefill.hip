// Causal Taylor linear attention over a whole sequence (prefill) for gfx950.
//
// Kernels behind the entry points:
//
//  * lin_prefill_mfma_kernel (bf16 in/out): chunked scan, 64 tokens per chunk, one workgroup
//    of FOUR wavefronts per (batch, head, 64-channel block).  The running state stays in MFMA
//    accumulators for the length of the sequence, split by feature slots over the four
//    wavefronts; a bf16 image of it goes through LDS once per chunk for the read-out, which is
//    split by tokens.  Small batches scan every sequence as concurrent segments (two passes of
//    this kernel around lin_prefill_prefix_kernel).
//
//      within a chunk   A = tril(1 + s + s^2/2), s = q.k/4, from a K=16 MFMA on the raw
//                       16-dim q, k (never expanding the features), then O^T += V^T A^T
//      across chunks    O^T += S^T psi(q)^T   and afterwards   S += psi(k)^T V
//
//    psi is a 160-slot SYMMETRIC packing of the 273 TaylorExp features (x_i x_j and x_j x_i
//    are one slot with doubled weight), laid out by circular distance t: slot (t, j) holds
//    x_j * x_{(j - t) mod 16} for t = 0..7; tile 8 holds the 8 distance-8 pairs, the constant
//    feature and 7 zeros; tile 9 the linear terms.  With that layout
//      - psi(k)^T (lane <-> slot, registers <-> tokens) is one DPP row-rotate multiply per
//        element, with the weights folded into a pre-scaled copy of k;
//      - psi(q)^T (lane <-> token, registers <-> slots) is a product of two registers with
//        compile-time indices, because each lane group keeps q rotated by 4*group.
//    The normaliser is carried as a 65th value channel of ones, so numerator and
//    denominator come out of the same MFMAs.  The in-chunk weights feed their product with V
//    straight from the accumulator registers (accumulator layout == B/A operand layout for a
//    product contracted over the accumulator's row index); V needs a transpose, done by the
//    transposing LDS read.  At the end the 160-slot state is expanded to the (dv, 273) decode
//    layout.
//
//  * lin_prefill_f32_kernel (fp32 or bf16 in/out, fp32 arithmetic throughout): a plain
//    recurrent evaluation, four tokens per round.  It serves fp32 callers (tolerance 1e-4
//    is out of reach of bf16 operands) and is an independent second implementation that
//    the tests compare the MFMA kernel against at sizes the CPU cannot reach.
#include <atomic>
#include <mutex>
#include <type_traits>
#include <utility>

#include "common.hpp"

namespace based {

// ------------------------------------------------------------------------------------------
// compile-time loop: body(std::integral_constant<int, I>{}) for I in [0, N)
// ------------------------------------------------------------------------------------------
template <int N, typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl<N>(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

template <int T>
__device__ __forceinline__ float row_ror(float x) {
  // value of lane (i - T) mod 16 within each row of 16 lanes
  static_assert(T >= 1 && T <= 15, "rotation out of range");
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x120 + T, 0xf, 0xf, false));
}

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

__device__ __forceinline__ bf16x8 pack8(const float (&x)[8]) {
  u32x4 w = {pack_bf16(x[0], x[1]), pack_bf16(x[2], x[3]), pack_bf16(x[4], x[5]), pack_bf16(x[6], x[7])};
  return __builtin_bit_cast(bf16x8, w);
}

__device__ __forceinline__ f32x4 mfma(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

constexpr int kChunk = 64;       // tokens per chunk
constexpr int kFTiles = 10;      // 160 symmetric feature slots = 10 tiles of 16 (see own_tile)
constexpr int kETiles = 5;       // 64 value channels + 1 normaliser channel (tile 4, column 0)
constexpr int kVStride = 80;     // bf16 per V row in LDS (64 channels + pad): 160 B rows make the
                                 // transposing reads below conflict-free
constexpr int kOStride = 72;     // bf16 per row of the output staging tile (64 channels + pad, 144 B)
constexpr float kSqrt2 = 1.4142135623730951f;

// Position of chunk-relative token tau inside a V^T row / inside the contraction slots:
// slab s = tau/32 holds, for lane group g, slots jj = 0..7 <-> tokens 32s + 16(jj/4) + 4g + jj%4,
// which is the order in which accumulator rows (4g + r of tiles 2s, 2s+1) turn into operand slots.
__device__ __forceinline__ int slot_token(int s, int g, int jj) {
  return 32 * s + 16 * (jj >> 2) + 4 * g + (jj & 3);
}

constexpr int kWavesPerChain = 4;   // wavefronts cooperating on one (batch, head, channel block)
// Slot tiles of the state owned by wavefront w: {0,1,2}, {3,4,5}, {6,7}, {8,9}.  The wavefronts
// with fewer slot tiles own the token tiles with more causal work (see the kernel), which
// balances the MFMA count per wavefront to 58..62 per chunk.
__host__ __device__ constexpr int own_count(int wave) { return wave < 2 ? 3 : 2; }
__host__ __device__ constexpr int own_tile(int wave, int i) { return (wave < 2 ? 3 * wave : 2 * wave + 2) + i; }
static_assert(own_tile(3, own_count(3) - 1) == kFTiles - 1, "slot tiles must be covered exactly");

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
constexpr int kSbBytes = 5 * kETiles * 64 * 16;   // bf16 image of the state: [slab][channel tile][lane] x 16 B

// The whole per-chain loop as seen by wavefront `wave` (a compile-time role: the four roles run
// different instruction streams, chosen by a scalar branch at kernel entry, and meet only at
// the workgroup barriers).
//
// MODE selects how much of a sequence one workgroup scans (small batches split each sequence
// into segments so that the whole GPU has work; see based_linear_attn_prefill_split):
//   kModeFull   the whole sequence, state starting at zero;
//   kModeDelta  tokens [t_begin, t_end) only, state update only (no outputs), state starting at
//               zero and dumped to the workspace at the end (the segment's contribution);
//   kModeFrom   tokens [t_begin, t_end) in full, state starting from the workspace entry (the
//               exclusive prefix over the earlier segments).
constexpr int kModeFull = 0, kModeDelta = 1, kModeFrom = 2;
constexpr int kSegStateFloats = kFTiles * kETiles * 64 * 4;  // accumulator image of one chain's state

template <int wave, int MODE>
__device__ __forceinline__ void lin_prefill_chain(
    __bf16* s_q, __bf16* s_k, __bf16* s_v, unsigned char* s_sb, __bf16* s_o,
    const __bf16* __restrict__ q, const __bf16* __restrict__ k, const __bf16* __restrict__ v,
    __bf16* __restrict__ y, float* __restrict__ kv_state, float* __restrict__ k_state, int H, int L,
    int dv, long q_sb, long q_sh, long q_sl, long k_sb, long k_sh, long k_sl, long v_sb, long v_sh,
    long v_sl, long y_sb, long y_sh, long y_sl, float eps, float* __restrict__ ws, int seg_tokens, int n_seg) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int col = lane & 15;
  const int grp = lane >> 4;
  // Workgroups are dealt to the 8 XCDs round-robin by workgroup id.  Chains whose q/k rows share
  // cache lines (neighbouring heads of one batch entry: 32-byte rows, 512 bytes apart) should
  // sit behind the same L2, so consecutive chain numbers are laid along one XCD:
  // chain = (id mod 8) * ceil(n / 8) + id / 8 when that stays in range.
  const long n_chain = gridDim.x;
  const long per_xcd = (n_chain + 7) / 8;
  long bh = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (n_chain % 8 != 0) bh = blockIdx.x;  // irregular grids keep the identity mapping
  const int eb = blockIdx.y;  // 64-channel block of the value dimension
  const int b = (int)(bh / H), h = (int)(bh % H);

  q += b * q_sb + h * q_sh;
  k += b * k_sb + h * k_sh;
  v += b * v_sb + h * v_sh + 64 * eb;
  y += b * y_sb + h * y_sh + 64 * eb;

  // Division of labour between the four wavefronts of a chain:
  //   read-out  (O^T = V^T A^T + S^T psi(q)^T)  split by TOKENS : wave w owns token tile w of the
  //             chunk and contracts it against the whole state;
  //   update    (S += psi(k)^T V)               split by SLOTS  : wave w owns slot tiles own_tile(w, .).
  // Each wavefront therefore generates every psi element exactly once, holds only its share of
  // the fp32 state in accumulators, and publishes a bf16 image of that share in LDS once per
  // chunk for the others' read-out.
  constexpr int kOwn = own_count(wave);

  // own share of the running state S[i <-> slot tile own_tile(wave, i)][channel tile]:
  // lane <-> channel 16 et + col, regs <-> slot positions 4 grp + r
  f32x4 S[kOwn][kETiles];
#pragma unroll
  for (int i = 0; i < kOwn; ++i)
#pragma unroll
    for (int et = 0; et < kETiles; ++et) S[i][et] = f32x4{0.f, 0.f, 0.f, 0.f};

  // token range of this workgroup and its slot in the workspace
  const int seg = blockIdx.z;
  const int t_begin = MODE == kModeFull ? 0 : seg * seg_tokens;
  const int t_end = MODE == kModeFull ? L : (t_begin + seg_tokens < L ? t_begin + seg_tokens : L);
  const bool last_seg = MODE == kModeFull || seg == n_seg - 1;
  float* ws_mine = nullptr;
  if constexpr (MODE != kModeFull)
    ws_mine = ws + (((long)bh * gridDim.y + eb) * n_seg + seg) * (long)kSegStateFloats;
  if constexpr (MODE == kModeFrom) {
#pragma unroll
    for (int i = 0; i < kOwn; ++i)
#pragma unroll
      for (int et = 0; et < kETiles; ++et)
        S[i][et] = *reinterpret_cast<const f32x4*>(ws_mine + ((own_tile(wave, i) * kETiles + et) * 64 + lane) * 4);
  }

  // operand of the normaliser channel: row/column 64 (col == 0) is all ones
  const uint32_t one2 = col == 0 ? 0x3F803F80u : 0u;
  const bf16x8 ones_op = __builtin_bit_cast(bf16x8, u32x4{one2, one2, one2, one2});
  const bool low_half = grp < 2;  // feature positions 4 grp + c < 8
  const uint32_t t8_keep = col < 8 ? 0xFFFFFFFFu : 0u;      // slot tile 8: pair products live in positions 0..7,
  const uint32_t t8_const = col == 8 ? 0x3F803F80u : 0u;    // the constant feature (bf16 1.0) in position 8

  // Global loads of a chunk, issued one phase ahead of their use.  q (wave 0) / k (wave 1):
  // 64 rows x 32 B, lane <-> row.  v: 64 rows x 128 B = 512 pieces of 16 B, two per thread:
  // piece 256 i + tid <-> (token piece / 8, channels 8 (piece % 8) ..+8).
  u32x4 pf_qk[2];
  bf16x8 pf_v[2];
  auto issue_loads = [&](int t0) {
    const int ntok = t_end - t0 < kChunk ? t_end - t0 : kChunk;
    if (ntok == kChunk) {  // whole chunk (all but possibly the last): no zero fill, no bounds
      if constexpr (wave == 1 || (wave == 0 && MODE != kModeDelta)) {
        const __bf16* base = wave == 0 ? q + (long)(t0 + lane) * q_sl : k + (long)(t0 + lane) * k_sl;
        const u32x4* src = reinterpret_cast<const u32x4*>(base);
        pf_qk[0] = src[0];
        pf_qk[1] = src[1];
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int piece = 256 * i + tid;
        pf_v[i] = *reinterpret_cast<const bf16x8*>(v + (long)(t0 + (piece >> 3)) * v_sl + 8 * (piece & 7));
      }
      return;
    }
    if constexpr (wave == 1 || (wave == 0 && MODE != kModeDelta)) {
      const u32x4 z4 = {0, 0, 0, 0};
      pf_qk[0] = pf_qk[1] = z4;
      if (lane < ntok) {
        const __bf16* base = wave == 0 ? q + (long)(t0 + lane) * q_sl : k + (long)(t0 + lane) * k_sl;
        const u32x4* src = reinterpret_cast<const u32x4*>(base);
        pf_qk[0] = src[0];
        pf_qk[1] = src[1];
      }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int piece = 256 * i + tid;
      const int tau = piece >> 3;
      bf16x8 x = {0, 0, 0, 0, 0, 0, 0, 0};
      if (tau < ntok) x = *reinterpret_cast<const bf16x8*>(v + (long)(t0 + tau) * v_sl + 8 * (piece & 7));
      pf_v[i] = x;
    }
  };
  if (t_begin < t_end) issue_loads(t_begin);

  // V^T operand tile (lane <-> channel 16 et + col, slots jj <-> tokens 32 s + 16 (jj/4) + 4 grp + jj%4)
  // straight from the row-major V chunk in LDS with the transposing 64-bit LDS read: inside
  // each group of 16 lanes, lane 4a + b receives element b of what lanes a, a+4, a+8, a+12
  // loaded, so source lane 4j + a fetches channels 4a..4a+3 of token j of the group's four.
  const __bf16* vt_base = s_v + (4 * grp + (col >> 2)) * kVStride + 4 * (col & 3);
  const __bf16* kt_base = s_k + (4 * grp + (col >> 2)) * kFeat + 4 * (col & 3);
  auto load_vt = [&](int et, int s) -> bf16x8 {
    const __bf16* p0 = vt_base + (32 * s) * kVStride + 16 * et;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)p0);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (s16x4 __attribute__((address_space(3)))*)(p0 + 16 * kVStride));
    const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(bf16x8, both);
  };

  for (int t0 = t_begin; t0 < t_end; t0 += kChunk) {
    const int ntok = t_end - t0 < kChunk ? t_end - t0 : kChunk;

    // ---------------- stage the chunk (q, k, v rows as they come) into LDS ----------------
    {
      if constexpr (wave == 1 || (wave == 0 && MODE != kModeDelta)) {
        u32x4* dst = reinterpret_cast<u32x4*>((wave == 0 ? s_q : s_k) + lane * kFeat);
        dst[0] = pf_qk[0];
        dst[1] = pf_qk[1];
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int piece = 256 * i + tid;
        *reinterpret_cast<bf16x8*>(s_v + (piece >> 3) * kVStride + 8 * (piece & 7)) = pf_v[i];
      }
    }
    // ---------------- publish the bf16 image of the own share of the state ----------------
    // s_sb[slab][channel tile][lane] is the 16-byte A operand of the read-out: bytes 0..7 come
    // from slot tile 2 slab (regs r = 0..3), bytes 8..15 from slot tile 2 slab + 1.
    // A wavefront that owns both slot tiles of a slab writes the operand in one 16-byte piece.
    if constexpr (MODE != kModeDelta) {
      static_for<kOwn>([&](auto II) {
        constexpr int i = decltype(II)::value;
        constexpr int t = own_tile(wave, i);
        constexpr bool pair_lo = (t % 2 == 0) && (i + 1 < kOwn);
        constexpr bool pair_hi = (t % 2 == 1) && (i > 0);
        if constexpr (pair_lo) {
#pragma unroll
          for (int et = 0; et < kETiles; ++et) {
            const u32x4 w4 = {pack_bf16(S[i][et][0], S[i][et][1]), pack_bf16(S[i][et][2], S[i][et][3]),
                              pack_bf16(S[i + 1][et][0], S[i + 1][et][1]), pack_bf16(S[i + 1][et][2], S[i + 1][et][3])};
            *reinterpret_cast<u32x4*>(s_sb + (((t >> 1) * kETiles + et) * 64 + lane) * 16) = w4;
          }
        } else if constexpr (!pair_hi) {
#pragma unroll
          for (int et = 0; et < kETiles; ++et) {
            const uint2 w2 = make_uint2(pack_bf16(S[i][et][0], S[i][et][1]), pack_bf16(S[i][et][2], S[i][et][3]));
            *reinterpret_cast<uint2*>(s_sb + (((t >> 1) * kETiles + et) * 64 + lane) * 16 + (t & 1) * 8) = w2;
          }
        }
      });
    }
    __syncthreads();

    // next chunk's global loads are in flight for the whole of this chunk's compute
    if (t0 + kChunk < t_end) issue_loads(t0 + kChunk);

    // ---------------- read-out of one own token tile: intra-chunk part, state part, store ----------------
    auto readout = [&](auto NT) {
      constexpr int nt = decltype(NT)::value;  // token tile within the chunk
      // O^T[channel tile]: lane <-> token 16 nt + col, regs <-> channel 4 grp + r
      f32x4 O[kETiles];
#pragma unroll
      for (int et = 0; et < kETiles; ++et) O[et] = f32x4{0.f, 0.f, 0.f, 0.f};

      // within the chunk: A^T = tril(1 + s + s^2/2)^T from a K=16 product of raw q, k; O^T += V^T A^T.
      {
        // the 16 features are exactly the contraction of a 16x16x16 MFMA: lane <-> (row, features 4 grp ..+3)
        const s16x4 bq = *reinterpret_cast<const s16x4*>(s_q + (16 * nt + col) * kFeat + 4 * grp);
        float p[4][4];  // [key tile][r]; tiles above the diagonal stay zero
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
          for (int r = 0; r < 4; ++r) p[mt][r] = 0.f;
        static_for<nt + 1>([&](auto MT) {
          constexpr int mt = decltype(MT)::value;
          const s16x4 ka = *reinterpret_cast<const s16x4*>(s_k + (16 * mt + col) * kFeat + 4 * grp);
          const f32x4 a = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ka, bq, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float pv = __builtin_fmaf(a[r], __builtin_fmaf(a[r], 1.0f / 32.0f, 0.25f), 1.0f);
            if (mt == nt) pv = (4 * grp + r <= col) ? pv : 0.f;  // key <= query on the diagonal tile
            p[mt][r] = pv;
          }
        });
        static_for<nt / 2 + 1>([&](auto SS) {
          constexpr int s = decltype(SS)::value;
          const float pb[8] = {p[2 * s][0], p[2 * s][1], p[2 * s][2], p[2 * s][3],
                               p[2 * s + 1][0], p[2 * s + 1][1], p[2 * s + 1][2], p[2 * s + 1][3]};
          const bf16x8 bp = pack8(pb);
#pragma unroll
          for (int et = 0; et < 4; ++et) O[et] = mfma(load_vt(et, s), bp, O[et]);
          O[4] = mfma(ones_op, bp, O[4]);
        });
      }

      // across chunks: O^T += S^T psi(q)^T with the state as it was before this chunk
      {
        // q of token 16 nt + col, rotated by 4 grp: qr[r] = q[(4 grp + r) mod 16]
        float qr[16];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const bf16x4 x = *reinterpret_cast<const bf16x4*>(s_q + (16 * nt + col) * kFeat + ((4 * grp + 4 * i) & 15));
#pragma unroll
          for (int c = 0; c < 4; ++c) qr[4 * i + c] = to_f32(x[c]);
        }
        const float fix8_0 = (grp == 2) ? 1.0f : 0.0f;  // slot (tile 8, position 8) = constant feature
        static_for<5>([&](auto SG) {
          constexpr int sg = decltype(SG)::value;  // slab of 32 slots = slot tiles 2 sg, 2 sg + 1
          float f[8];
          static_for<8>([&](auto JJ) {
            constexpr int jj = decltype(JJ)::value;
            constexpr int t = 2 * sg + jj / 4;  // slot tile
            constexpr int c = jj % 4;           // position 4 grp + c
            const float own = qr[c];
            if constexpr (t == 0) {
              f[jj] = own * own;
            } else if constexpr (t <= 7) {
              f[jj] = own * qr[(c - t) & 15];
            } else if constexpr (t == 8) {
              const float prod = own * qr[(c - 8) & 15];
              f[jj] = low_half ? prod : (c == 0 ? fix8_0 : 0.0f);
            } else {
              f[jj] = own;
            }
          });
          const bf16x8 bq = pack8(f);
#pragma unroll
          for (int et = 0; et < kETiles; ++et) {
            const bf16x8 sa = *reinterpret_cast<const bf16x8*>(s_sb + ((sg * kETiles + et) * 64 + lane) * 16);
            O[et] = mfma(sa, bq, O[et]);
          }
        });
      }

      // normalise: the denominator sits in lane group 0, register 0 of channel tile 4
      const float z = __shfl(O[4][0], col, 64);
      const float inv = 1.0f / (z + eps);
      // store: the 16 x 64 output tile goes through a wave-private LDS tile so that each lane
      // writes 16 contiguous bytes and 8 lanes cover one 128-byte row (8-byte scattered stores
      // cost four times the L2 write requests)
      __bf16* so = s_o + wave * (16 * kOStride);
#pragma unroll
      for (int et = 0; et < 4; ++et) {
        const uint32_t w0 = pack_bf16(O[et][0] * inv, O[et][1] * inv);
        const uint32_t w1 = pack_bf16(O[et][2] * inv, O[et][3] * inv);
        *reinterpret_cast<uint2*>(so + col * kOStride + 16 * et + 4 * grp) = make_uint2(w0, w1);
      }
      // the tile is re-read below in another lane layout: order the wavefront's own LDS accesses
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int hlf = 0; hlf < 2; ++hlf) {
        const int row = 8 * hlf + (lane >> 3);
        const u32x4 w4 = *reinterpret_cast<const u32x4*>(so + row * kOStride + 8 * (lane & 7));
        const int tau = 16 * nt + row;
        if (tau < ntok) *reinterpret_cast<u32x4*>(y + (long)(t0 + tau) * y_sl + 8 * (lane & 7)) = w4;
      }
    };
    if constexpr (MODE != kModeDelta) readout(std::integral_constant<int, wave>{});
    __builtin_amdgcn_sched_barrier(0);

    // ---------------- state update: S += psi(k)^T V for the own slot tiles ----------------
    {
      // lane <-> slot position j = col; registers <-> the 8 token slots of a slab.  One slab of
      // 32 tokens at a time, so that only its k values and V^T tiles are live.
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        float kraw[8], k16[8];
        bf16x8 vt[4];
        {
          // k^T (lane <-> feature col, slots <-> tokens) with the same transposing read as V^T
          const __bf16* p0 = kt_base + (32 * s) * kFeat;
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)p0);
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (s16x4 __attribute__((address_space(3)))*)(p0 + 16 * kFeat));
#pragma unroll
          for (int jj = 0; jj < 8; ++jj) {
            const uint32_t bits = (uint32_t)(uint16_t)(jj < 4 ? lo[jj & 3] : hi[jj & 3]) << 16;
            const float x = __builtin_bit_cast(float, bits);
            kraw[jj] = x;
            k16[jj] = x * (1.0f / 16.0f);
          }
        }
#pragma unroll
        for (int et = 0; et < 4; ++et) vt[et] = load_vt(et, s);
        static_for<kOwn>([&](auto II) {
          constexpr int i = decltype(II)::value;
          constexpr int t = own_tile(wave, i);  // slot tile
          float f[8];
#pragma unroll
          for (int jj = 0; jj < 8; ++jj) {
            if constexpr (t == 0) {
              f[jj] = kraw[jj] * k16[jj] * 0.5f;
            } else if constexpr (t <= 7) {
              f[jj] = row_ror<t>(kraw[jj]) * k16[jj];
            } else if constexpr (t == 8) {
              f[jj] = row_ror<8>(kraw[jj]) * k16[jj];  // positions 8..15 are replaced below
            } else {
              f[jj] = kraw[jj] * 0.25f;
            }
          }
          bf16x8 ak = pack8(f);
          if constexpr (t == 8) {
            // position 8 is the constant feature, 9..15 are unused.  The constant is also set
            // for the zero rows that pad the last chunk: their v is zero, and the count they
            // add to the normaliser state is taken off when the state is written out.
            u32x4 w = __builtin_bit_cast(u32x4, ak);
#pragma unroll
            for (int d = 0; d < 4; ++d) w[d] = (w[d] & t8_keep) | t8_const;
            ak = __builtin_bit_cast(bf16x8, w);
          }
#pragma unroll
          for (int et = 0; et < 4; ++et) S[i][et] = mfma(ak, vt[et], S[i][et]);
          S[i][4] = mfma(ak, ones_op, S[i][4]);
        });
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __syncthreads();  // LDS is overwritten by the next chunk
  }

  // ---------------- a segment's contribution goes to the workspace as it sits in registers ----------------
  if constexpr (MODE == kModeDelta) {
#pragma unroll
    for (int i = 0; i < kOwn; ++i)
#pragma unroll
      for (int et = 0; et < kETiles; ++et)
        *reinterpret_cast<f32x4*>(ws_mine + ((own_tile(wave, i) * kETiles + et) * 64 + lane) * 4) = S[i][et];
    return;
  }

  // ---------------- expand the 160-slot state into the (dv, 273) decode layout ----------------
  // Sixteen channels at a time: the four wavefronts scatter their slot tiles of one channel
  // tile into a 16 x 273 fp32 block in LDS (each cross slot lands on both (i, j) and (j, i),
  // with the factor that undoes the packing weights), and the block, which is contiguous in
  // the decode state, leaves with coalesced 16-byte stores.
  if (kv_state != nullptr && last_seg) {
    const int pad_tokens = (kChunk - (t_end - t_begin) % kChunk) % kChunk;
    float* blk = reinterpret_cast<float*>(s_sb);
    static_assert(16 * kExp * 4 <= kSbBytes, "expansion block must fit in the state image buffer");
    static_for<kETiles>([&](auto ET) {
      constexpr int et = decltype(ET)::value;
      __syncthreads();  // the buffer is free (main loop done / previous block copied out)
      float* row = blk + col * kExp;
      static_for<kOwn>([&](auto II) {
        constexpr int i = decltype(II)::value;
        constexpr int t = own_tile(wave, i);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int j = 4 * grp + r;
          const float x = S[i][et][r];
          if constexpr (t == 0) {
            row[1 + kFeat + 17 * j] = x * (4.0f * kSqrt2);
          } else if constexpr (t <= 7) {
            const int pj = (j - t) & 15;
            row[1 + kFeat + 16 * j + pj] = x * (2.0f * kSqrt2);
            row[1 + kFeat + 16 * pj + j] = x * (2.0f * kSqrt2);
          } else if constexpr (t == 8) {
            if (j < 8) {
              row[1 + kFeat + 16 * j + j + 8] = x * (2.0f * kSqrt2);
              row[1 + kFeat + 16 * (j + 8) + j] = x * (2.0f * kSqrt2);
            } else if (j == 8) {
              // constant feature; in the normaliser column it counted the padding rows too
              row[0] = et == 4 ? x - (float)pad_tokens : x;
            }
          } else {
            row[1 + j] = x * 2.0f;
          }
        }
      });
      __syncthreads();
      if constexpr (et < 4) {
        f32x4* dst = reinterpret_cast<f32x4*>(kv_state + (bh * dv + 64 * eb + 16 * et) * kExp);
        const f32x4* src = reinterpret_cast<const f32x4*>(blk);
        for (int idx = tid; idx < 16 * kExp / 4; idx += 64 * kWavesPerChain) dst[idx] = src[idx];
      } else if (eb == 0) {
        // channel tile 4 carries the normaliser state in its column 0 (= row 0 of the block)
        for (int idx = tid; idx < kExp; idx += 64 * kWavesPerChain) k_state[bh * kExp + idx] = blk[idx];
      }
    });
  }
}

template <int MODE>
__global__ __launch_bounds__(64 * kWavesPerChain, 3) void lin_prefill_mfma_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ k, const __bf16* __restrict__ v,
    __bf16* __restrict__ y, float* __restrict__ kv_state, float* __restrict__ k_state, int H, int L,
    int dv, long q_sb, long q_sh, long q_sl, long k_sb, long k_sh, long k_sl, long v_sb, long v_sh,
    long v_sl, long y_sb, long y_sh, long y_sl, float eps, float* __restrict__ ws, int seg_tokens, int n_seg) {
  __shared__ __align__(16) __bf16 s_q[kChunk * kFeat];
  __shared__ __align__(16) __bf16 s_k[kChunk * kFeat];
  __shared__ __align__(16) __bf16 s_v[kChunk * kVStride];
  __shared__ __align__(16) unsigned char s_sb[kSbBytes];
  __shared__ __align__(16) __bf16 s_o[kWavesPerChain * 16 * kOStride];
#define BASED_CHAIN_ARGS s_q, s_k, s_v, s_sb, s_o, q, k, v, y, kv_state, k_state, H, L, dv, q_sb, q_sh, q_sl, k_sb, k_sh, \
                         k_sl, v_sb, v_sh, v_sl, y_sb, y_sh, y_sl, eps, ws, seg_tokens, n_seg
  switch (__builtin_amdgcn_readfirstlane(threadIdx.x >> 6)) {
    case 0: lin_prefill_chain<0, MODE>(BASED_CHAIN_ARGS); break;
    case 1: lin_prefill_chain<1, MODE>(BASED_CHAIN_ARGS); break;
    case 2: lin_prefill_chain<2, MODE>(BASED_CHAIN_ARGS); break;
    default: lin_prefill_chain<3, MODE>(BASED_CHAIN_ARGS); break;
  }
#undef BASED_CHAIN_ARGS
}

// In-place exclusive prefix over the segments of each chain: ws[c][s] <- sum_{s' < s} ws[c][s'].
// The last segment's entry is never produced by the delta pass and is treated as zero.
__global__ __launch_bounds__(256) void lin_prefill_prefix_kernel(float* __restrict__ ws, int n_seg) {
  float* base = ws + (long)blockIdx.x * n_seg * kSegStateFloats;
  const int idx = blockIdx.y * blockDim.x + threadIdx.x;  // one float4 of the state image per thread
  if (idx >= kSegStateFloats / 4) return;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  // eight segments at a time: the loads are independent, only the running sum is sequential
  for (int s0 = 0; s0 < n_seg; s0 += 8) {
    f32x4 cur[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      cur[u] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (s0 + u < n_seg - 1) cur[u] = reinterpret_cast<const f32x4*>(base + (long)(s0 + u) * kSegStateFloats)[idx];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (s0 + u < n_seg) reinterpret_cast<f32x4*>(base + (long)(s0 + u) * kSegStateFloats)[idx] = acc;
      acc += cur[u];
    }
  }
}

// ------------------------------------------------------------------------------------------
// fp32-arithmetic recurrent kernel.  Workgroup = (b, h, 64-channel block), 256 threads:
// thread (e = tid % 64, fg = tid / 64) owns state entries S[f][e] for f = 4 i + fg.
// ------------------------------------------------------------------------------------------
constexpr int kRound = 4;                       // tokens per synchronisation round
constexpr int kOwn = (kExp + 3) / 4;            // 69 state entries per thread

__device__ __forceinline__ float phi_full(const float* x, int f) {
  if (f == 0) return 1.0f;
  if (f <= kFeat) return x[f - 1] * 0.5f;
  const int g = f - 1 - kFeat;
  return x[g >> 4] * x[g & 15] * 0.17677669529663687f;
}

template <typename T>
__global__ __launch_bounds__(256) void lin_prefill_f32_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, T* __restrict__ y,
    float* __restrict__ kv_state, float* __restrict__ k_state, int H, int L, int dv, long q_sb,
    long q_sh, long q_sl, long k_sb, long k_sh, long k_sl, long v_sb, long v_sh, long v_sl,
    long y_sb, long y_sh, long y_sl, float eps) {
  __shared__ float s_x[kRound][2][kFeat];          // [token][0 = k, 1 = q]
  __shared__ float s_v[kRound][64];
  __shared__ float s_phi[kRound][2][kExp + 3];
  __shared__ float s_part[kRound][4][64];
  __shared__ float s_den[kRound][4];

  const int tid = threadIdx.x;
  const int e = tid & 63, fg = tid >> 6;
  const long bh = blockIdx.x;
  const int eb = blockIdx.y;
  const int b = (int)(bh / H), h = (int)(bh % H);
  const int ew = dv - 64 * eb < 64 ? dv - 64 * eb : 64;  // live channels in this block
  q += b * q_sb + h * q_sh;
  k += b * k_sb + h * k_sh;
  v += b * v_sb + h * v_sh + 64 * eb;
  y += b * y_sb + h * y_sh + 64 * eb;

  float S[kOwn];
#pragma unroll
  for (int i = 0; i < kOwn; ++i) S[i] = 0.f;
  float ks0 = 0.f, ks1 = 0.f;  // normaliser state for features tid and tid + 256

  for (int t0 = 0; t0 < L; t0 += kRound) {
    const int nt = L - t0 < kRound ? L - t0 : kRound;
    if (tid < kRound * 2 * kFeat) {
      const int tt = tid / (2 * kFeat), which = (tid / kFeat) & 1, i = tid % kFeat;
      float x = 0.f;
      if (tt < nt) x = to_f32((which ? q : k)[(long)(t0 + tt) * (which ? q_sl : k_sl) + i]);
      s_x[tt][which][i] = x;
    }
    {
      const int tt = tid >> 6;
      float x = 0.f;
      if (tt < nt && e < ew) x = to_f32(v[(long)(t0 + tt) * v_sl + e]);
      s_v[tt][e] = x;
    }
    __syncthreads();
    for (int idx = tid; idx < kRound * 2 * kExp; idx += 256) {
      const int tt = idx / (2 * kExp), rem = idx % (2 * kExp);
      const int which = rem / kExp, f = rem % kExp;
      s_phi[tt][which][f] = phi_full(s_x[tt][which], f);
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float ve = s_v[tt][e];
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < kOwn; ++i) {
        const int f = 4 * i + fg;
        if (f < kExp) {
          S[i] = __builtin_fmaf(s_phi[tt][0][f], ve, S[i]);
          acc = __builtin_fmaf(s_phi[tt][1][f], S[i], acc);
        }
      }
      s_part[tt][fg][e] = acc;
      ks0 += s_phi[tt][0][tid];
      float dpart = s_phi[tt][1][tid] * ks0;
      if (tid + 256 < kExp) {
        ks1 += s_phi[tt][0][tid + 256];
        dpart = __builtin_fmaf(s_phi[tt][1][tid + 256], ks1, dpart);
      }
      dpart = wave_sum(dpart);
      if (e == 0) s_den[tt][fg] = dpart;
    }
    __syncthreads();
    {
      const int tt = tid >> 6;
      if (tt < nt && e < ew) {
        const float num = s_part[tt][0][e] + s_part[tt][1][e] + s_part[tt][2][e] + s_part[tt][3][e];
        const float den = s_den[tt][0] + s_den[tt][1] + s_den[tt][2] + s_den[tt][3];
        y[(long)(t0 + tt) * y_sl + e] = from_f32<T>(num / (den + eps));
      }
    }
    __syncthreads();
  }

  if (kv_state != nullptr) {
    if (e < ew) {
      float* row = kv_state + (bh * dv + 64 * eb + e) * kExp;
#pragma unroll
      for (int i = 0; i < kOwn; ++i) {
        const int f = 4 * i + fg;
        if (f < kExp) row[f] = S[i];
      }
    }
    if (eb == 0) {
      k_state[bh * kExp + tid] = ks0;
      if (tid + 256 < kExp) k_state[bh * kExp + tid + 256] = ks1;
    }
  }
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace based

extern "C" BASED_API int based_linear_attn_prefill(
    const void* q, const void* k, const void* v, void* y, float* kv_state, float* k_state, int64_t B,
    int64_t H, int64_t L, int64_t dv, int64_t q_sb, int64_t q_sh, int64_t q_sl, int64_t k_sb,
    int64_t k_sh, int64_t k_sl, int64_t v_sb, int64_t v_sh, int64_t v_sl, int64_t y_sb, int64_t y_sh,
    int64_t y_sl, float eps, int io_dtype, void* stream) {
  using namespace based;
  BASED_REQUIRE(q && k && v && y, BASED_ERR_ARG, "linear_attn_prefill: null pointer argument");
  BASED_REQUIRE((kv_state == nullptr) == (k_state == nullptr), BASED_ERR_ARG,
                "linear_attn_prefill: kv_state and k_state must both be given or both be NULL");
  BASED_REQUIRE(B >= 0 && H > 0 && L >= 0, BASED_ERR_ARG, "linear_attn_prefill: bad sizes");
  BASED_REQUIRE(io_dtype == BASED_BF16 || io_dtype == BASED_F32, BASED_ERR_DTYPE,
                "linear_attn_prefill: io_dtype %d unsupported", io_dtype);
  BASED_REQUIRE(B * H < (1ll << 31) && L < (1ll << 31), BASED_ERR_SHAPE, "linear_attn_prefill: sizes too large");
  if (B == 0) return BASED_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (io_dtype == BASED_BF16 && (dv == 64 || dv == 128)) {
    const int64_t strides[] = {q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, y_sb, y_sh, y_sl};
    for (int64_t st : strides)
      BASED_REQUIRE(st % 8 == 0, BASED_ERR_ALIGN,
                    "linear_attn_prefill: bf16 strides must be multiples of 8 elements (16 bytes)");
    BASED_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(y), BASED_ERR_ALIGN,
                  "linear_attn_prefill: tensors must be 16-byte aligned");
    dim3 grid((unsigned)(B * H), (unsigned)(dv / 64)), block(64 * kWavesPerChain);
    hipLaunchKernelGGL(lin_prefill_mfma_kernel<kModeFull>, grid, block, 0, s, (const __bf16*)q, (const __bf16*)k,
                       (const __bf16*)v, (__bf16*)y, kv_state, k_state, (int)H, (int)L, (int)dv, q_sb,
                       q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, y_sb, y_sh, y_sl, eps, (float*)nullptr, 0, 1);
    return check_launch("linear_attn_prefill");
  }
  BASED_REQUIRE(dv >= 1 && dv <= 1024, BASED_ERR_SHAPE, "linear_attn_prefill: head dim %ld unsupported",
                (long)dv);
  dim3 grid((unsigned)(B * H), (unsigned)((dv + 63) / 64)), block(256);
  if (io_dtype == BASED_BF16) {
    hipLaunchKernelGGL(lin_prefill_f32_kernel<__bf16>, grid, block, 0, s, (const __bf16*)q,
                       (const __bf16*)k, (const __bf16*)v, (__bf16*)y, kv_state, k_state, (int)H, (int)L,
                       (int)dv, q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, y_sb, y_sh, y_sl, eps);
  } else {
    hipLaunchKernelGGL(lin_prefill_f32_kernel<float>, grid, block, 0, s, (const float*)q,
                       (const float*)k, (const float*)v, (float*)y, kv_state, k_state, (int)H, (int)L,
                       (int)dv, q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, y_sb, y_sh, y_sl, eps);
  }
  return check_launch("linear_attn_prefill");
}

// Workgroup slots of one full wave of the MFMA prefill kernel on MI355X (256 CUs x 3 resident
// workgroups); segment counts are chosen to fill about one such wave.
static constexpr int64_t kPrefillSlots = 768;

extern "C" BASED_API int based_linear_attn_prefill_plan(int64_t B, int64_t H, int64_t L, int64_t dv,
                                                        int io_dtype, int64_t* n_seg,
                                                        int64_t* workspace_bytes) {
  using namespace based;
  BASED_REQUIRE(n_seg && workspace_bytes, BASED_ERR_ARG, "linear_attn_prefill_plan: null output pointer");
  *n_seg = 1;
  *workspace_bytes = 0;
  if (io_dtype != BASED_BF16 || (dv != 64 && dv != 128) || B <= 0 || H <= 0 || L <= 0) return BASED_OK;
  const int64_t chains = B * H * (dv / 64);
  const int64_t chunks = (L + kChunk - 1) / kChunk;
  if (chains * 3 >= kPrefillSlots * 2 || chunks < 2) return BASED_OK;  // enough chains already
  int64_t want = (kPrefillSlots + chains - 1) / chains;
  if (want > chunks) want = chunks;
  int64_t seg_chunks = (chunks + want - 1) / want;
  // a segment costs about three chunks' worth of fixed work (loading its prefix, dumping or
  // expanding its state): below four chunks per segment more segments stop paying
  if (seg_chunks < 4) seg_chunks = chunks < 4 ? chunks : 4;
  const int64_t segs = (chunks + seg_chunks - 1) / seg_chunks;
  if (segs < 2) return BASED_OK;
  *n_seg = segs;
  *workspace_bytes = chains * segs * (int64_t)kSegStateFloats * 4;
  return BASED_OK;
}

namespace based {

// Validation and the three launches of the segmented scan, shared by the entry point that is
// handed a workspace and the one that uses the library's own static scratch array.
static int launch_prefill_split(const char* who, const void* q, const void* k, const void* v, void* y,
                                float* kv_state, float* k_state, int64_t B, int64_t H, int64_t L, int64_t dv,
                                int64_t q_sb, int64_t q_sh, int64_t q_sl, int64_t k_sb, int64_t k_sh, int64_t k_sl,
                                int64_t v_sb, int64_t v_sh, int64_t v_sl, int64_t y_sb, int64_t y_sh, int64_t y_sl,
                                float eps, int io_dtype, int64_t n_seg, void* workspace, int64_t workspace_bytes,
                                int64_t workspace_limit, void* stream) {
  BASED_REQUIRE(q && k && v && y, BASED_ERR_ARG, "%s: null pointer argument", who);
  BASED_REQUIRE((kv_state == nullptr) == (k_state == nullptr), BASED_ERR_ARG,
                "%s: kv_state and k_state must both be given or both be NULL", who);
  BASED_REQUIRE(io_dtype == BASED_BF16 && (dv == 64 || dv == 128), BASED_ERR_SHAPE,
                "%s: only the bf16 MFMA path (dv 64 or 128) can be split", who);
  BASED_REQUIRE(B > 0 && H > 0 && L > 0 && B * H < (1ll << 31) && L < (1ll << 31), BASED_ERR_ARG, "%s: bad sizes", who);
  const int64_t chunks = (L + kChunk - 1) / kChunk;
  BASED_REQUIRE(n_seg >= 2 && n_seg <= chunks && n_seg < 65536, BASED_ERR_ARG, "%s: %ld segments for %ld chunks", who,
                (long)n_seg, (long)chunks);
  const int64_t seg_chunks = (chunks + n_seg - 1) / n_seg;
  BASED_REQUIRE((n_seg - 1) * seg_chunks < chunks, BASED_ERR_ARG,
                "%s: segment count %ld leaves empty segments (use the plan)", who, (long)n_seg);
  const int64_t chains = B * H * (dv / 64);
  const int64_t need = chains * n_seg * (int64_t)kSegStateFloats * 4;
  if (workspace_limit >= 0)
    BASED_REQUIRE(need <= workspace_limit, BASED_ERR_SHAPE,
                  "%s: %ld chains x %ld segments need %ld bytes of scratch, the static array holds %ld", who,
                  (long)chains, (long)n_seg, (long)need, (long)workspace_limit);
  BASED_REQUIRE(workspace != nullptr, BASED_ERR_ARG, "%s: null workspace", who);
  BASED_REQUIRE(workspace_bytes >= need, BASED_ERR_ARG, "%s: workspace too small", who);
  const int64_t strides[] = {q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, y_sb, y_sh, y_sl};
  for (int64_t st : strides)
    BASED_REQUIRE(st % 8 == 0, BASED_ERR_ALIGN, "%s: bf16 strides must be multiples of 8 elements (16 bytes)", who);
  BASED_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(y) && aligned16(workspace),
                BASED_ERR_ALIGN, "%s: tensors must be 16-byte aligned", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* ws = static_cast<float*>(workspace);
  const int seg_tokens = (int)(seg_chunks * kChunk);
  dim3 block(64 * kWavesPerChain);
  // pass 1: every segment but the last accumulates its own contribution to the state
  hipLaunchKernelGGL(lin_prefill_mfma_kernel<kModeDelta>, dim3((unsigned)(B * H), (unsigned)(dv / 64), (unsigned)(n_seg - 1)),
                     block, 0, s, (const __bf16*)q, (const __bf16*)k, (const __bf16*)v, (__bf16*)y, kv_state,
                     k_state, (int)H, (int)L, (int)dv, q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, y_sb,
                     y_sh, y_sl, eps, ws, seg_tokens, (int)n_seg);
  int rc = check_launch(who);
  if (rc) return rc;
  hipLaunchKernelGGL(lin_prefill_prefix_kernel, dim3((unsigned)chains, (kSegStateFloats / 4 + 255) / 256), dim3(256), 0, s,
                     ws, (int)n_seg);
  rc = check_launch(who);
  if (rc) return rc;
  hipLaunchKernelGGL(lin_prefill_mfma_kernel<kModeFrom>, dim3((unsigned)(B * H), (unsigned)(dv / 64), (unsigned)n_seg),
                     block, 0, s, (const __bf16*)q, (const __bf16*)k, (const __bf16*)v, (__bf16*)y, kv_state,
                     k_state, (int)H, (int)L, (int)dv, q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, y_sb,
                     y_sh, y_sl, eps, ws, seg_tokens, (int)n_seg);
  return check_launch(who);
}

// Scratch of based_linear_attn_prefill_split_static: one array per GPU, part of the code object,
// alive until the process ends.  64 MiB hold 1310 (chain, segment) state images, more than any
// segment count the plan entry point returns (it aims at 768 workgroup slots and never exceeds
// 1150 images).  In host code the array's name is only a handle for hipGetSymbolAddress; the
// device address is looked up once per device and kept in g_scratch_ptr.
constexpr int64_t kStaticScratchBytes = BASED_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char g_split_scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

// Device address of the current device's copy of the scratch array (nullptr + error set on failure).
static void* static_scratch_for_current_device(const char* who) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("%s: cannot identify the current device (%s)", who, e != hipSuccess ? hipGetErrorString(e) : "index out of range");
    return nullptr;
  }
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p != nullptr) return p;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p != nullptr) return p;
  e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_split_scratch));
  if (e != hipSuccess || p == nullptr) {
    set_error("%s: hipGetSymbolAddress of the scratch array failed on device %d: %s", who, dev, hipGetErrorString(e));
    return nullptr;
  }
  g_scratch_ptr[dev].store(p, std::memory_order_release);
  return p;
}

}  // namespace based

extern "C" BASED_API int based_linear_attn_prefill_split(
    const void* q, const void* k, const void* v, void* y, float* kv_state, float* k_state, int64_t B,
    int64_t H, int64_t L, int64_t dv, int64_t q_sb, int64_t q_sh, int64_t q_sl, int64_t k_sb,
    int64_t k_sh, int64_t k_sl, int64_t v_sb, int64_t v_sh, int64_t v_sl, int64_t y_sb, int64_t y_sh,
    int64_t y_sl, float eps, int io_dtype, int64_t n_seg, void* workspace, int64_t workspace_bytes,
    void* stream) {
  if (n_seg <= 1)
    return based_linear_attn_prefill(q, k, v, y, kv_state, k_state, B, H, L, dv, q_sb, q_sh, q_sl, k_sb, k_sh,
                                     k_sl, v_sb, v_sh, v_sl, y_sb, y_sh, y_sl, eps, io_dtype, stream);
  return based::launch_prefill_split("linear_attn_prefill_split", q, k, v, y, kv_state, k_state, B, H, L, dv, q_sb,
                                     q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, y_sb, y_sh, y_sl, eps, io_dtype,
                                     n_seg, workspace, workspace_bytes, -1, stream);
}

extern "C" BASED_API int based_linear_attn_prefill_split_static(
    const void* q, const void* k, const void* v, void* y, float* kv_state, float* k_state, int64_t B,
    int64_t H, int64_t L, int64_t dv, int64_t q_sb, int64_t q_sh, int64_t q_sl, int64_t k_sb,
    int64_t k_sh, int64_t k_sl, int64_t v_sb, int64_t v_sh, int64_t v_sl, int64_t y_sb, int64_t y_sh,
    int64_t y_sl, float eps, int io_dtype, int64_t n_seg, void* stream) {
  using namespace based;
  if (n_seg <= 1)  // the unsplit kernel has no scratch at all
    return based_linear_attn_prefill(q, k, v, y, kv_state, k_state, B, H, L, dv, q_sb, q_sh, q_sl, k_sb, k_sh,
                                     k_sl, v_sb, v_sh, v_sl, y_sb, y_sh, y_sl, eps, io_dtype, stream);
  // size check first: an oversized request is refused without touching the device
  if (io_dtype == BASED_BF16 && (dv == 64 || dv == 128) && B > 0 && H > 0)
    BASED_REQUIRE(B * H * (dv / 64) * n_seg * (int64_t)kSegStateFloats * 4 <= kStaticScratchBytes, BASED_ERR_SHAPE,
                  "linear_attn_prefill_split_static: %ld chains x %ld segments need %ld bytes of scratch, the "
                  "static array holds %ld",
                  (long)(B * H * (dv / 64)), (long)n_seg, (long)(B * H * (dv / 64) * n_seg * (int64_t)kSegStateFloats * 4),
                  (long)kStaticScratchBytes);
  void* scratch = static_scratch_for_current_device("linear_attn_prefill_split_static");
  if (scratch == nullptr) return BASED_ERR_LAUNCH;
  return launch_prefill_split("linear_attn_prefill_split_static", q, k, v, y, kv_state, k_state, B, H, L, dv, q_sb,
                              q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, y_sb, y_sh, y_sl, eps, io_dtype, n_seg,
                              scratch, kStaticScratchBytes, kStaticScratchBytes, stream);
}
