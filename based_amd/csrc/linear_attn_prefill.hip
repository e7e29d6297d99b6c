// Causal Taylor linear attention over a whole sequence (prefill) for gfx950.
//
// Kernels behind the entry points:
//
//  * lin_prefill_mfma_kernel (bf16 in/out): chunked scan, 64 tokens per chunk, one workgroup
//    of EIGHT wavefronts per (batch, head, 64-channel block) -- or per (batch, head) with both
//    blocks when the head dim is 65..128 --: four updaters keep the running
//    state in MFMA accumulators for the length of the sequence, split by feature slots, and
//    publish a bf16 image of it in LDS once per chunk; four readers, split by tokens, compute
//    the outputs from the chunk's rows and the image.  Small batches scan every sequence as
//    concurrent segments (two passes of this kernel around lin_prefill_prefix_kernel).
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
//    The normaliser is a quadratic form in the raw q over the first and second moments of k
//    (see below), not a 65th value channel.  The in-chunk weights feed their product with V
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
constexpr int kCTiles = 4;       // 64 value channels = 4 tiles of 16
constexpr float kSqrt2 = 1.4142135623730951f;

// Position of chunk-relative token tau inside a V^T row / inside the contraction slots:
// slab s = tau/32 holds, for lane group g, slots jj = 0..7 <-> tokens 32s + 16(jj/4) + 4g + jj%4,
// which is the order in which accumulator rows (4g + r of tiles 2s, 2s+1) turn into operand slots.
__device__ __forceinline__ int slot_token(int s, int g, int jj) {
  return 32 * s + 16 * (jj >> 2) + 4 * g + (jj & 3);
}

constexpr int kWavesPerChain = 4;   // wavefronts cooperating on one (batch, head, channel block)
// Slot tiles of the state owned by updater w, in the order it works through them: {0,1,2},
// {4,5,3}, {6,7}, {8,9}.  The first two are always the two tiles of one 32-slot slab (their bf16
// image leaves as one 16-byte piece per lane); updaters 0 and 1 share slab 1.  Updater
// kNormWave also carries the normaliser state.
__host__ __device__ constexpr int own_count(int wave) { return wave < 2 ? 3 : 2; }
__host__ __device__ constexpr int own_tile(int wave, int i) {
  return wave == 0 ? i : wave == 1 ? (i < 2 ? 4 + i : 3) : 2 * wave + 2 + i;
}
static_assert(own_tile(3, own_count(3) - 1) == kFTiles - 1 && own_tile(1, 2) == 3 && own_tile(0, 2) == 2 &&
                  own_tile(2, 0) == 6, "slot tiles must be covered exactly");
constexpr int kNormWave = 2;

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;

// LDS of one workgroup (80,000 B: two workgroups per compute unit).
//   data ring, 3 slots : the q, k, v rows of a chunk, written by direct global->LDS loads two
//                        chunks ahead of their use (no registers, HBM latency fully covered).
//                        q, k: 64 rows x 32 B, the two 16-byte halves of a row swapped when
//                        bit 2 of the row index is set (column reads of 8 bytes from 16
//                        consecutive rows then hit 8 distinct bank pairs instead of 4).
//                        v: 64 rows x 128 B whose eight 16-byte pieces
//                        are stored at piece index p ^ 2 (row & 3), which makes the transposing
//                        reads below bank-conflict free without row padding (a direct load
//                        writes the 64 lanes' pieces back to back, so rows cannot be padded).
//   state image, 2     : bf16 image of the state, [slab][channel tile][lane] x 16 B; chunk c is
//                        read out from image[c & 1] while image[(c+1) & 1] is being written.
//   K2, K1, 2 each     : normaliser state (see below).
// A workgroup carries CT channel tiles of its head: 4 (one block of 64 channels; two workgroups
// per compute unit) or 8 (two blocks; head dims 65..128: psi(q) and psi(k) are generated once for
// both blocks, at 142 KB of LDS and up to 256 registers, i.e. one workgroup per compute unit).
// With two blocks the v rows of a ring slot are two 64 x 128 B arrays, one per block, each laid
// out as described above.  CTL <= CT of the tiles are live: for head dims 97..112 (112 is the
// released 1B / 1.3B shape) the eighth tile's products, operand reads and image stores are
// compiled out (the layouts keep eight tiles; B=4, L=4096, dv=112: 63 -> 59 us; large batches wait
// for their rows and gain nothing).
constexpr int kRing = 3;
constexpr int kQkBytes = kChunk * kFeat * 2;       // 2 KB
constexpr int kVBlockBytes = kChunk * 64 * 2;      // 8 KB: the v rows of one block of 64 channels
constexpr int kDataK = kQkBytes, kDataV = 2 * kQkBytes;
constexpr int kK2Bytes = 2 * 64 * 8;               // hi and lo halves of the 16x16 second-moment operand
constexpr int kOffData = 0;
template <int CT>
struct PrefillLds {
  static_assert(CT == 4 || CT == 8, "one or two blocks of 64 channels");
  static constexpr int kBlocks = CT / 4;
  static constexpr int kDataBytes = 2 * kQkBytes + kBlocks * kVBlockBytes;  // one ring slot: q | k | v
  static constexpr int kImgBytes = 5 * CT * 64 * 16;   // state image: [slab][channel tile][lane] x 16 B
  static constexpr int kOffImg = kOffData + kRing * kDataBytes;
  static constexpr int kOffK2 = kOffImg + 2 * kImgBytes;
  static constexpr int kOffK1 = kOffK2 + 2 * kK2Bytes;      // [2][16] floats: first moment of k
  static constexpr int kBytes = kOffK1 + 2 * 16 * 4;
  // of the wave-wide direct loads of a chunk (q 2, k 2, v 8 per block) each updater issues
  static constexpr int kLoadsPerUpdater = (4 + 8 * kBlocks) / kWavesPerChain;
  static_assert(kOffImg % 16 == 0 && kOffK2 % 16 == 0 && kOffK1 % 16 == 0, "16-byte aligned sections");
  static_assert(kBytes * (CT == 4 ? 2 : 1) <= 160 * 1024, "must fit the 160 KB of a compute unit");
};

// One chain = one (batch, head, 64-channel block); a workgroup scans one chain, or the two chains
// of a head with 65..128 channels side by side (CT = 8 channel tiles: every per-tile array below
// is twice as long, the roles and the stages are the same).  The scan runs in chunks of 64 tokens
// on EIGHT wavefronts in two kinds of roles that run concurrently and meet at one barrier per
// chunk:
//   readers  (wavefronts 0..3, one per token tile of the chunk): O^T = V^T A^T + S^T psi(q)^T, the
//            normaliser, the division and the store.  They read the chunk's rows and the bf16
//            image of the state as it was before the chunk.
//   updaters (wavefronts 4..7, each owning slot tiles own_tile(w, .)): stage the next chunk's rows
//            into LDS, request the rows after that, S += psi(k)^T V in fp32 accumulators, and
//            publish the bf16 image of the new state for the next chunk's readers.
// A SIMD hosts one reader and one updater of each resident workgroup, so the vector work of one
// role runs under the MFMAs of the other.  Every psi element is generated exactly once.
//
// MODE selects how much of a sequence one workgroup scans (small batches split each sequence
// into segments so that the whole GPU has work; see based_linear_attn_prefill_split):
//   kModeFull   the whole sequence, state starting at zero;
//   kModeDelta  tokens [t_begin, t_end) only, state update only (no outputs), state starting at
//               zero and dumped to the workspace at the end (the segment's contribution);
//   kModeFrom   tokens [t_begin, t_end) in full, state starting from the workspace entry (the
//               exclusive prefix over the earlier segments, made by lin_prefill_prefix_kernel);
//   kModeFromSum  the same, but the workspace still holds the segments' own contributions and
//               the workgroup adds up the earlier ones itself (few segments: saves a launch).
//
// The normaliser z_i = sum_{j<=i} (1 + s_ij + s_ij^2/2), s_ij = q_i.k_j/4, is NOT carried as a
// 65th value channel.  Over the earlier chunks it is the quadratic form
//   N + q_i.K1/4 + q_i^T K2 q_i/32,  N = number of earlier tokens, K1 = sum_j k_j, K2 = sum_j k_j k_j^T,
// which costs one MFMA on the raw q (K2 as a hi + lo pair of bf16 operands) and four
// multiply-adds per lane; inside the chunk it is the row sum of the in-chunk weights.  K2 is one
// 16x16 accumulator tile (two MFMAs per chunk on the k^T operand that psi(k) is generated from).
constexpr int kModeFull = 0, kModeDelta = 1, kModeFrom = 2, kModeFromSum = 3;
// One chain's state as it goes through the workspace of the segmented scan: the accumulator image
// of S (slot tile, channel tile, lane, 4), then the accumulators of K2 and of K1 (lane, 4 each).
constexpr int kSegStateFloats = BASED_PREFILL_SEGMENT_STATE_BYTES / 4;
constexpr int kWsK2 = kFTiles * kCTiles * 256;
constexpr int kWsK1 = kWsK2 + 256;
static_assert(kWsK1 + 256 == kSegStateFloats, "workspace layout");
constexpr int kThreads = 64 * 2 * kWavesPerChain;  // 4 readers + 4 updaters

// sum over the four lane groups (lanes col, col+16, col+32, col+48); every lane gets the total
__device__ __forceinline__ float group_allreduce(float x) {
  x += __shfl_xor(x, 16, 64);
  x += __shfl_xor(x, 32, 64);
  return x;
}

// The loop bodies below are written as sequences of STAGES.  A stage first issues the LDS reads
// for the operands of the next stage, then runs its own group of MFMAs interleaved with the
// vector instructions that build the next stage's register operand (psi(q) or psi(k) tiles, the
// in-chunk weights), so that neither LDS latency nor the vector work sits between two MFMAs of
// one wavefront.  sched_barrier pins the stage boundaries, sched_group_barrier the interleave.
#define BASED_STAGE_END() __builtin_amdgcn_sched_barrier(0)
// NM groups of (1 MFMA, NV vector instructions); the rest of the region floats behind
template <int NM, int NV>
__device__ __forceinline__ void interleave() {
  static_for<NM>([](auto) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x002, NV, 0);
  });
}

#define BASED_CHAIN_PARAMS                                                                                          \
  unsigned char *lds, const __bf16 *__restrict__ q, const __bf16 *__restrict__ k, const __bf16 *__restrict__ v,      \
      __bf16 *__restrict__ y, float *__restrict__ kv_state, float *__restrict__ k_state, int H, int L, int dv,       \
      long q_sb, long q_sh, long q_sl, long k_sb, long k_sh, long k_sl, long v_sb, long v_sh, long v_sl, long y_sb,  \
      long y_sh, long y_sl, float eps, float *__restrict__ ws, int seg_tokens, int n_seg

// Work item of this workgroup: item = (batch * H + head) * n_wb + workgroup of the head, n_wb =
// ceil(dv / 64) workgroups of one channel block each, or 1 that carries both blocks (prefill_item).  Workgroups are dealt to the 8 XCDs round-robin by workgroup id.  Items whose rows
// share cache lines (the channel blocks of one head read the same q and k rows, and for head dims
// that are no multiple of 64 their v and y rows meet inside 128-byte lines; neighbouring heads of
// one batch entry: 32-byte q / k rows 512 bytes apart) should sit behind the same L2 at about the
// same time, so consecutive items are laid along one XCD: item = (id mod 8) * ceil(n / 8) + id / 8
// when that stays in range.
__device__ __forceinline__ long item_of_block() {
  const long n_item = gridDim.x;
  const long per_xcd = (n_item + 7) / 8;
  if (n_item % 8 != 0) return blockIdx.x;  // irregular grids keep the identity mapping
  return (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
}

// What a workgroup works on: head `bh`, its first block of 64 channels `eb0`, how many of the
// workgroup's channels exist (`live`, a multiple of 16), and the index of that first block among
// all (head, block) chains (the unit of the segmented scan's workspace).
struct PrefillItem {
  long bh, chain0;
  int eb0, live;
};
template <int CT>
__device__ __forceinline__ PrefillItem prefill_item(int dv) {
  constexpr int kBlocks = CT / 4;
  const int n_eb = (dv + 63) >> 6;
  const int n_wb = (n_eb + kBlocks - 1) / kBlocks;  // workgroups per head
  const long item = item_of_block();
  PrefillItem it;
  it.bh = item / n_wb;
  it.eb0 = (int)(item % n_wb) * kBlocks;
  it.live = dv - 64 * it.eb0 < 64 * kBlocks ? dv - 64 * it.eb0 : 64 * kBlocks;
  it.chain0 = it.bh * n_eb + it.eb0;
  return it;
}

// Transposing 64-bit LDS read pair: inside each group of 16 lanes, lane 4a + b receives element
// b of what lanes a, a+4, a+8, a+12 loaded.  `p` is the lane's source address for the first four
// tokens; the second four are `hi_bytes` further on.
__device__ __forceinline__ bf16x8 load_tr_pair(const unsigned char* p, int hi_bytes) {
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)p);
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p + hi_bytes));
  const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(bf16x8, both);
}
// V^T operand tile of channel tile et, token slab s (lane <-> channel 16 et + col, slots jj <->
// tokens 32 s + 16 (jj/4) + 4 grp + jj%4) from the swizzled V rows of a ring slot: source lane
// 4j + a of a group fetches channels 16 et + 4a..+3 of token 32 s + 4 grp + j (+16), which sit in
// 16-byte piece (2 et + a/2) ^ 2j of the row, i.e. at byte ((et ^ j) << 5) + 8a.
// vt_lane = 128 (4 grp + j) + 8a is the lane's part of the address.
// Channel tiles 4 and up belong to the second block of 64 channels, whose rows follow the first's.
__device__ __forceinline__ bf16x8 load_vt(const unsigned char* slot, int vt_lane, int j, int et, int s) {
  return load_tr_pair(slot + kDataV + (et >> 2) * kVBlockBytes + vt_lane + (((et ^ j) & 3) << 5) + 4096 * s, 2048);
}
// k^T operand tile of token slab s (lane <-> feature col) from the row-major 32-byte k rows
__device__ __forceinline__ bf16x8 load_kt(const unsigned char* slot, int kt_lane, int s) {
  return load_tr_pair(slot + kDataK + kt_lane + 1024 * s, 512);
}

// Workgroup barriers of the chunk loop.  __syncthreads() would make an updater wait for ALL of
// its outstanding direct global->LDS loads, including the ones requested two chunks ahead, so
// the two roles use narrower forms:
//  * readers only touch LDS: a workgroup fence restricted to the LDS address space;
//  * updaters spell the waits out: own LDS traffic done (lgkmcnt 0), and all but the newest
//    `newest` direct loads landed (vmcnt); s_waitcnt immediates are gfx9-encoded
//    (vmcnt[3:0] | expcnt 7 << 4 | lgkmcnt << 8).
__device__ __forceinline__ void barrier_reader() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
template <int newest>
__device__ __forceinline__ void barrier_updater() {
  static_assert(newest >= 0 && newest < 16, "vmcnt immediate");
  __builtin_amdgcn_s_waitcnt(0x0070 | newest);
  __builtin_amdgcn_s_barrier();
}

// ------------------------------------------------------------------------------------------
// reader of token tile nt
// ------------------------------------------------------------------------------------------
template <int nt, int MODE, int CT, int CTL>
__device__ __forceinline__ void lin_prefill_reader(BASED_CHAIN_PARAMS) {
  using LD = PrefillLds<CT>;
  const int lane = threadIdx.x & 63;
  const int col = lane & 15;
  const int grp = lane >> 4;
  const PrefillItem it = prefill_item<CT>(dv);
  const long bh = it.bh;
  const int eb = it.eb0;        // first 64-channel block of this workgroup
  const int live_ch = it.live;  // channels of this workgroup that exist (a multiple of 16)
  const int b = (int)(bh / H), h = (int)(bh % H);
  y += b * y_sb + h * y_sh + 64 * eb;
  const int seg = blockIdx.z;
  const int t_begin = MODE == kModeFull ? 0 : seg * seg_tokens;
  const int t_end = MODE == kModeFull ? L : (t_begin + seg_tokens < L ? t_begin + seg_tokens : L);
  const bool last_seg = MODE == kModeFull || seg == n_seg - 1;
  const bool low_half = grp < 2;  // feature positions 4 grp + c < 8
  const int vt_j = col >> 2;
  const int vt_lane = 128 * (4 * grp + vt_j) + 8 * (col & 3);
  const int qk_swz = (col >> 2) & 1 ? 2 : 0;  // rows 16 x + col: bit 2 of the row index swaps the halves
  // output: after the lane-group exchange below a lane owns 2 x 8 consecutive channels of its token
  const int out_ch = (grp & 1) * 32 + 4 * (grp & 2);
  using std::integral_constant;

  barrier_reader();  // chunk 0 and the initial state are staged
  int slot_i = 0, buf = 0;
  for (int t0 = t_begin; t0 < t_end; t0 += kChunk, buf ^= 1, slot_i = slot_i == kRing - 1 ? 0 : slot_i + 1) {
    if constexpr (MODE != kModeDelta) {
      const int ntok = t_end - t0 < kChunk ? t_end - t0 : kChunk;
      const unsigned char* slot = lds + kOffData + slot_i * LD::kDataBytes;
      const __bf16* s_q = reinterpret_cast<const __bf16*>(slot);
      const __bf16* s_k = reinterpret_cast<const __bf16*>(slot + kDataK);
      const unsigned char* s_img = lds + LD::kOffImg + buf * LD::kImgBytes;

      // O^T[channel tile]: lane <-> token 16 nt + col, regs <-> channel 4 grp + r
      f32x4 O[CT];
#pragma unroll
      for (int et = 0; et < CT; ++et) O[et] = f32x4{0.f, 0.f, 0.f, 0.f};

      // ---- reads of the first stages ----
      // the 16 raw features are exactly the contraction of a 16x16x16 MFMA: lane <-> (row, features 4 grp ..+3)
      // (feature chunk c of a row sits at 8-byte position c ^ qk_swz of that row)
      const s16x4 bq = *reinterpret_cast<const s16x4*>(s_q + (16 * nt + col) * kFeat + 4 * (grp ^ qk_swz));
      bf16x4 qx[4];  // q of token 16 nt + col, rotated by 4 grp
#pragma unroll
      for (int i = 0; i < 4; ++i)
        qx[i] = *reinterpret_cast<const bf16x4*>(s_q + (16 * nt + col) * kFeat + 4 * (((grp + i) & 3) ^ qk_swz));
      const unsigned char* k2 = lds + LD::kOffK2 + buf * kK2Bytes;
      const s16x4 k2hi = *reinterpret_cast<const s16x4*>(k2 + lane * 8);
      const s16x4 k2lo = *reinterpret_cast<const s16x4*>(k2 + 512 + lane * 8);
      const f32x4 k1 = *reinterpret_cast<const f32x4*>(lds + LD::kOffK1 + buf * 64 + 16 * grp);
      s16x4 ka[nt + 1];
#pragma unroll
      for (int mt = 0; mt <= nt; ++mt)
        ka[mt] = *reinterpret_cast<const s16x4*>(s_k + (16 * mt + col) * kFeat + 4 * (grp ^ qk_swz));
      auto img_load = [&](int sg, bf16x8 (&A)[CT]) {
#pragma unroll
        for (int et = 0; et < CTL; ++et)
          A[et] = *reinterpret_cast<const bf16x8*>(s_img + ((sg * CT + et) * 64 + lane) * 16);
      };
      bf16x8 A[5][CT];
      img_load(0, A[0]);
      BASED_STAGE_END();

      // ---- qr[r] = q[(4 grp + r) mod 16] as floats ----
      float qr[16];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) qr[4 * i + c] = to_f32(qx[i][c]);
      const float fix8_0 = (grp == 2) ? 1.0f : 0.0f;  // slot (tile 8, position 8) = constant feature
      auto psi_q = [&](auto SG) -> bf16x8 {
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
        return pack8(f);
      };
      BASED_STAGE_END();

      // ---- stage Z: normaliser product and in-chunk scores (raw q, k operands) | psi(q) slab 0 ----
      // normaliser over the earlier chunks: U = K2 q with K2 = hi + lo (one K=32 MFMA over [hi | lo] x [q; q])
      const s16x8 k2both = {k2hi[0], k2hi[1], k2hi[2], k2hi[3], k2lo[0], k2lo[1], k2lo[2], k2lo[3]};
      const s16x8 bqbq = {bq[0], bq[1], bq[2], bq[3], bq[0], bq[1], bq[2], bq[3]};
      const f32x4 u = mfma(__builtin_bit_cast(bf16x8, k2both), __builtin_bit_cast(bf16x8, bqbq), f32x4{0.f, 0.f, 0.f, 0.f});
      f32x4 a[nt + 1];
#pragma unroll
      for (int mt = 0; mt <= nt; ++mt)
        a[mt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ka[mt], bq, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
      bf16x8 Bq[5];
      Bq[0] = psi_q(integral_constant<int, 0>{});
      interleave<nt + 2, 3>();
      BASED_STAGE_END();

      // ---- stages R0..R4: O^T += S^T psi(q)^T, slab by slab | next psi(q) slab, in-chunk weights ----
      // this lane's share of the normaliser of token 16 nt + col: first the quadratic form over
      // the earlier chunks, then the row sums of the in-chunk weights
      float zpart = 0.f;
      bf16x8 vt_p[2][CT];
      bf16x8 bp[2];
      // in-chunk weights 1 + s + s^2/2 (s = a/4) of key tiles 2 s, 2 s + 1, masked on the diagonal
      // tile, packed as the B operand of the V^T A^T product; tiles above the diagonal are zero
      auto weights = [&](auto SS) {
        constexpr int s = decltype(SS)::value;
        float pb[8];
        static_for<2>([&](auto HH) {
          constexpr int mt = 2 * s + decltype(HH)::value;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float pv = 0.f;
            if constexpr (mt <= nt) {
              pv = __builtin_fmaf(a[mt][r], __builtin_fmaf(a[mt][r], 1.0f / 32.0f, 0.25f), 1.0f);
              if (mt == nt) pv = (4 * grp + r <= col) ? pv : 0.f;  // key <= query on the diagonal tile
              zpart += pv;
            }
            pb[4 * decltype(HH)::value + r] = pv;
          }
        });
        bp[s] = pack8(pb);
      };
      static_for<5>([&](auto SG) {
        constexpr int sg = decltype(SG)::value;
        if constexpr (sg + 1 < 5) img_load(sg + 1, A[sg + 1]);
        if constexpr (sg == 3) {
#pragma unroll
          for (int et = 0; et < CTL; ++et) vt_p[0][et] = load_vt(slot, vt_lane, vt_j, et, 0);
        }
        if constexpr (sg == 4 && nt >= 2) {
#pragma unroll
          for (int et = 0; et < CTL; ++et) vt_p[1][et] = load_vt(slot, vt_lane, vt_j, et, 1);
        }
#pragma unroll
        for (int et = 0; et < CTL; ++et) O[et] = mfma(A[sg][et], Bq[sg], O[et]);
        if constexpr (sg + 1 < 5) Bq[sg + 1] = psi_q(integral_constant<int, sg + 1>{});
        if constexpr (sg == 0) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            zpart = __builtin_fmaf(qr[r], __builtin_fmaf(u[r], 1.0f / 32.0f, k1[r] * 0.25f), zpart);
          weights(integral_constant<int, 0>{});
        }
        if constexpr (sg == 1 && nt >= 2) weights(integral_constant<int, 1>{});
        interleave<CTL, ((sg == 0 ? 9 : (sg == 1 && nt >= 2) ? 8 : 3) * 4 + CTL - 1) / CTL>();
        BASED_STAGE_END();
      });

      // ---- stages P0, P1: O^T += V^T A^T | the normaliser ----
      float inv = 0.f;
      static_for<nt / 2 + 1>([&](auto SS) {
        constexpr int s = decltype(SS)::value;
#pragma unroll
        for (int et = 0; et < CTL; ++et) O[et] = mfma(vt_p[s][et], bp[s], O[et]);
        if constexpr (s == 0) {
          // the earlier tokens count 1 each, the lane groups hold partial sums of the rest
          const float z = group_allreduce(zpart) + (float)t0;
          inv = __builtin_amdgcn_rcpf(z + eps);
        }
        BASED_STAGE_END();
      });

      // ---- normalise and store ----
      // A lane holds 4 channels (8 bytes) of each channel tile.  Lane groups g and g ^ 1 trade two
      // tiles (one row swap per dword), after which every lane holds 2 x 8 consecutive channels
      // and stores 16 contiguous bytes twice, straight from registers.
      uint32_t P[CT][2];
#pragma unroll
      for (int et = 0; et < CT; ++et) {
        if (et < CTL) {
          P[et][0] = pack_bf16(O[et][0] * inv, O[et][1] * inv);
          P[et][1] = pack_bf16(O[et][2] * inv, O[et][3] * inv);
        } else {
          P[et][0] = P[et][1] = 0;  // a tile past the head dim: never stored
        }
      }
      // The swap must not read a register in the two issue slots after a vector instruction wrote
      // it; the compiler does not look into inline assembly, so each one carries the wait.
#pragma unroll
      for (int blk = 0; blk < CT / 4; ++blk)
#pragma unroll
        for (int e = 0; e < 2; ++e)
#pragma unroll
          for (int d = 0; d < 2; ++d)
            asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(P[4 * blk + e][d]), "+v"(P[4 * blk + e + 2][d]));
      {
        const int tau = 16 * nt + col;
        if (tau < ntok) {
          // (channels past dv, in the last block of a head dim that is no multiple of 64, were
          // computed from stand-in data and are dropped here)
#pragma unroll
          for (int blk = 0; blk < CT / 4; ++blk) {
            const int ch = 64 * blk + out_ch;
            __bf16* dst = y + (long)(t0 + tau) * y_sl + ch;
            if (ch + 8 <= live_ch)
              *reinterpret_cast<u32x4*>(dst) = u32x4{P[4 * blk][0], P[4 * blk][1], P[4 * blk + 2][0], P[4 * blk + 2][1]};
            if (ch + 24 <= live_ch)
              *reinterpret_cast<u32x4*>(dst + 16) = u32x4{P[4 * blk + 1][0], P[4 * blk + 1][1], P[4 * blk + 3][0], P[4 * blk + 3][1]};
          }
        }
      }
    }
    barrier_reader();  // the next chunk's rows and state image are complete
  }

  // the updaters expand the state into the decode layout; readers help to copy it out
  if constexpr (MODE != kModeDelta) {
    if (kv_state != nullptr && last_seg) {
      const float* blk = reinterpret_cast<const float*>(lds + LD::kOffImg);
#pragma unroll 1
      for (int et = 0; 16 * et < live_ch; ++et) {
        __syncthreads();
        __syncthreads();
        f32x4* dst = reinterpret_cast<f32x4*>(kv_state + (bh * dv + 64 * eb + 16 * et) * kExp);
        const f32x4* src = reinterpret_cast<const f32x4*>(blk);
        for (int idx = threadIdx.x; idx < 16 * kExp / 4; idx += kThreads) dst[idx] = src[idx];
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// updater owning slot tiles own_tile(w, .)
// ------------------------------------------------------------------------------------------
template <int w, int MODE, int CT, int CTL>
__device__ __forceinline__ void lin_prefill_updater(BASED_CHAIN_PARAMS) {
  using LD = PrefillLds<CT>;
  constexpr int kLoads = LD::kLoadsPerUpdater;
  const int tid = threadIdx.x - 64 * kWavesPerChain;  // 0..255 among the updaters
  const int lane = tid & 63;
  const int col = lane & 15;
  const int grp = lane >> 4;
  const PrefillItem it = prefill_item<CT>(dv);
  const long bh = it.bh;
  const int eb = it.eb0;        // first 64-channel block of this workgroup
  const int live_ch = it.live;  // channels of this workgroup that exist (a multiple of 16)
  const int b = (int)(bh / H), h = (int)(bh % H);
  q += b * q_sb + h * q_sh;
  k += b * k_sb + h * k_sh;
  v += b * v_sb + h * v_sh + 64 * eb;
  constexpr int kOwn = own_count(w);
  constexpr bool kNorm = w == kNormWave;
  using std::integral_constant;

  // own share of the running state S[i <-> slot tile own_tile(w, i)][channel tile]:
  // lane <-> channel 16 et + col, regs <-> slot positions 4 grp + r
  f32x4 S[kOwn][CT];
#pragma unroll
  for (int i = 0; i < kOwn; ++i)
#pragma unroll
    for (int et = 0; et < CT; ++et) S[i][et] = f32x4{0.f, 0.f, 0.f, 0.f};
  // normaliser state (updater kNormWave only), both as MFMA accumulators:
  // K2[4 grp + r][col] (= K2[col][4 grp + r]) and K1[4 grp + r] (the same in every column)
  f32x4 K2 = {0.f, 0.f, 0.f, 0.f};
  f32x4 K1 = {0.f, 0.f, 0.f, 0.f};

  // token range of this workgroup and its slot in the workspace
  const int seg = blockIdx.z;
  const int t_begin = MODE == kModeFull ? 0 : seg * seg_tokens;
  const int t_end = MODE == kModeFull ? L : (t_begin + seg_tokens < L ? t_begin + seg_tokens : L);
  const bool last_seg = MODE == kModeFull || seg == n_seg - 1;
  // workspace entry of this segment for the workgroup's first block; the second block's chain
  // follows n_seg entries further on
  float* ws_mine = nullptr;
  if constexpr (MODE != kModeFull)
    ws_mine = ws + (it.chain0 * n_seg + seg) * (long)kSegStateFloats;
  const long ws_block = (long)n_seg * kSegStateFloats;
  // offset of accumulator tile (slot tile t, channel tile et) inside the workspace
  auto ws_tile = [&](int t, int et) { return (et >> 2) * ws_block + ((t * kCTiles + (et & 3)) * 64 + lane) * 4; };
  if constexpr (MODE == kModeFrom) {
#pragma unroll
    for (int i = 0; i < kOwn; ++i)
#pragma unroll
      for (int et = 0; et < CTL; ++et)
        S[i][et] = *reinterpret_cast<const f32x4*>(ws_mine + ws_tile(own_tile(w, i), et));
    if constexpr (kNorm) {
      K2 = *reinterpret_cast<const f32x4*>(ws_mine + kWsK2 + lane * 4);
      K1 = *reinterpret_cast<const f32x4*>(ws_mine + kWsK1 + lane * 4);
    }
  }
  if constexpr (MODE == kModeFromSum) {
    // same order of additions as lin_prefill_prefix_kernel: ((0 + d_0) + d_1) + ...
    const float* src = ws_mine - (long)seg * kSegStateFloats;
    for (int sp = 0; sp < seg; ++sp, src += kSegStateFloats) {
#pragma unroll
      for (int i = 0; i < kOwn; ++i)
#pragma unroll
        for (int et = 0; et < CTL; ++et)
          S[i][et] += *reinterpret_cast<const f32x4*>(src + ws_tile(own_tile(w, i), et));
      if constexpr (kNorm) {
        K2 += *reinterpret_cast<const f32x4*>(src + kWsK2 + lane * 4);
        K1 += *reinterpret_cast<const f32x4*>(src + kWsK1 + lane * 4);
      }
    }
  }

  const uint32_t t8_keep = col < 8 ? 0xFFFFFFFFu : 0u;      // slot tile 8: pair products live in positions 0..7,
  const uint32_t t8_const = col == 8 ? 0x3F803F80u : 0u;    // the constant feature (bf16 1.0) in position 8
  const bf16x8 ones8 = __builtin_bit_cast(bf16x8, u32x4{0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u});
  const int vt_j = col >> 2;
  const int vt_lane = 128 * (4 * grp + vt_j) + 8 * (col & 3);
  const int kt_lane = 32 * (4 * grp + vt_j) + 8 * ((col & 3) ^ (2 * (grp & 1)));  // rows 4 grp + j: bit 2 = grp & 1

  // Direct global->LDS loads of a chunk.  The twelve wave-wide loads of a chunk (64 lanes x 16 B
  // each, landing back to back in LDS) are dealt three to an updater: load id 0,1 = q rows 0..31,
  // 32..63 (lane <-> row id*32 + lane/2, LDS half lane%2 = global half (lane%2) ^ bit 2 of the
  // row); 2,3 = k likewise; 4 + j = v rows 8j..8j+7
  // (lane <-> row 8j + lane/8, LDS piece lane%8 = global piece (lane%8) ^ 2((lane/8) & 3)).
  // Rows past the end of the sequence are zero-filled instead.
  auto issue_loads = [&](int tc, int slot_index) {
    unsigned char* slot = lds + kOffData + slot_index * LD::kDataBytes;
    const int ntok = t_end - tc < kChunk ? t_end - tc : kChunk;
    static_for<kLoads>([&](auto II) {
      constexpr int id = kLoads * w + decltype(II)::value;
      if constexpr (MODE == kModeDelta && id < 2) return;  // no read-out, no q
      int row;
      const __bf16* src;
      unsigned char* dst;
      if constexpr (id < 4) {
        row = 32 * (id & 1) + (lane >> 1);
        src = (id < 2 ? q + (long)(tc + row) * q_sl : k + (long)(tc + row) * k_sl) + 8 * ((lane & 1) ^ ((lane >> 3) & 1));
        dst = slot + (id < 2 ? 0 : kDataK) + 1024 * (id & 1);
      } else {
        constexpr int vb = (id - 4) / 8, j = (id - 4) % 8;  // block of 64 channels, group of 8 rows
        row = 8 * j + (lane >> 3);
        // a piece past the head dim (last block of a dv that is no multiple of 64) is fetched from
        // piece 0 instead: channels are independent, so what such channels compute touches no
        // other, and they are never stored
        const int piece = (lane & 7) ^ (2 * ((lane >> 3) & 3));
        const int ch = 64 * vb + 8 * piece;
        src = v + (long)(tc + row) * v_sl + (ch < live_ch ? ch : 0);
        dst = slot + kDataV + vb * kVBlockBytes + 1024 * j;
      }
      if (ntok == kChunk || row < ntok) {
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                         (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
      } else {
        *reinterpret_cast<u32x4*>(dst + 16 * lane) = u32x4{0, 0, 0, 0};
      }
    });
  };
  // bf16 image of the own share of the state into image buffer `buf`.  img[slab][channel tile]
  // [lane] is the 16-byte A operand of the read-out: bytes 0..7 come from slot tile 2 slab (regs
  // r = 0..3), bytes 8..15 from slot tile 2 slab + 1.  The first two own tiles make up one slab
  // and leave as whole 16-byte pieces; a third tile fills its half of the shared slab.
  auto publish_pair = [&](int buf) {
    constexpr int t = own_tile(w, 0);
    static_assert(t % 2 == 0 && own_tile(w, 1) == t + 1, "first two own tiles = one slab");
    unsigned char* img = lds + LD::kOffImg + buf * LD::kImgBytes;
#pragma unroll
    for (int et = 0; et < CTL; ++et) {
      const u32x4 w4 = {pack_bf16(S[0][et][0], S[0][et][1]), pack_bf16(S[0][et][2], S[0][et][3]),
                        pack_bf16(S[1][et][0], S[1][et][1]), pack_bf16(S[1][et][2], S[1][et][3])};
      *reinterpret_cast<u32x4*>(img + (((t >> 1) * CT + et) * 64 + lane) * 16) = w4;
    }
  };
  auto publish_single = [&](int buf) {
    if constexpr (kOwn == 3) {
      constexpr int t = own_tile(w, 2);
      unsigned char* img = lds + LD::kOffImg + buf * LD::kImgBytes;
#pragma unroll
      for (int et = 0; et < CTL; ++et) {
        const uint2 w2 = make_uint2(pack_bf16(S[2][et][0], S[2][et][1]), pack_bf16(S[2][et][2], S[2][et][3]));
        *reinterpret_cast<uint2*>(img + (((t >> 1) * CT + et) * 64 + lane) * 16 + (t & 1) * 8) = w2;
      }
    }
  };
  auto publish_norm = [&](int buf) {
    if constexpr (kNorm) {
      // K2 as hi + lo bf16 operands: the accumulator registers K2[4 grp + r][col] are, by the
      // symmetry of K2, the A operand K2[m = col][k = 4 grp + r] of the readers' MFMA
      const uint32_t h0 = pack_bf16(K2[0], K2[1]), h1 = pack_bf16(K2[2], K2[3]);
      const float l0 = K2[0] - bf16_bits_to_f32(h0 & 0xFFFFu), l1 = K2[1] - __builtin_bit_cast(float, h0 & 0xFFFF0000u);
      const float l2 = K2[2] - bf16_bits_to_f32(h1 & 0xFFFFu), l3 = K2[3] - __builtin_bit_cast(float, h1 & 0xFFFF0000u);
      unsigned char* k2 = lds + LD::kOffK2 + buf * kK2Bytes;
      *reinterpret_cast<uint2*>(k2 + lane * 8) = make_uint2(h0, h1);
      *reinterpret_cast<uint2*>(k2 + 512 + lane * 8) = make_uint2(pack_bf16(l0, l1), pack_bf16(l2, l3));
      if (col == 0) *reinterpret_cast<f32x4*>(lds + LD::kOffK1 + buf * 64 + 16 * grp) = K1;
    }
  };

  // ---------------- prologue: chunks 0 and 1 requested, initial state published ----------------
  if (t_begin < t_end) issue_loads(t_begin, 0);
  if (t_begin + kChunk < t_end) issue_loads(t_begin + kChunk, 1);
  if constexpr (MODE != kModeDelta) {
    publish_pair(0);
    publish_single(0);
    publish_norm(0);
  }
  // Chunk 0 has landed; chunk 1 may stay in flight when it is a whole chunk (a partial chunk may
  // issue fewer loads than counted on, so then everything is awaited).
  constexpr int kInFlight = (MODE == kModeDelta && w == 0) ? kLoads - 2 : kLoads;  // this wavefront's loads per chunk
  if (t_begin + 2 * kChunk <= t_end) {
    barrier_updater<kInFlight>();
  } else {
    barrier_updater<0>();
  }

  int slot_i = 0, buf = 0;
  for (int t0 = t_begin; t0 < t_end; t0 += kChunk, buf ^= 1, slot_i = slot_i == kRing - 1 ? 0 : slot_i + 1) {
    const unsigned char* slot = lds + kOffData + slot_i * LD::kDataBytes;
    // operands of the first stage
    bf16x8 kt0 = load_kt(slot, kt_lane, 0);
    bf16x8 vt_s0[CT], vt_s1[CT];
#pragma unroll
    for (int et = 0; et < CTL; ++et) vt_s0[et] = load_vt(slot, vt_lane, vt_j, et, 0);
    // the rows of the chunk after the next are requested (their slot was last read one chunk ago)
    const bool more2 = t0 + 2 * kChunk < t_end;
    if (more2) issue_loads(t0 + 2 * kChunk, slot_i == 0 ? 2 : slot_i - 1);
    BASED_STAGE_END();

    // psi(k)^T tile (slot tile own_tile(w, i), current slab) from the raw k^T values of the slab;
    // lane <-> slot position col, registers <-> the slab's 8 token slots
    float k4[8];  // k / 4 of the slab's tokens (weights 1/16 on cross terms, 1/32 on squares, 1/4 on linear terms)
    auto psi_k = [&](auto II) -> bf16x8 {
      constexpr int t = own_tile(w, decltype(II)::value);
      bf16x8 ak;
      if constexpr (t == 9) {
        ak = pack8(k4);
      } else {
        float f[8];
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) {
          if constexpr (t == 0) {
            f[jj] = k4[jj] * k4[jj] * 0.5f;
          } else {
            f[jj] = row_ror<t>(k4[jj]) * k4[jj];  // tile 8: positions 8..15 are replaced below
          }
        }
        ak = pack8(f);
      }
      if constexpr (t == 8) {
        // position 8 is the constant feature, 9..15 are unused.  The constant is also set
        // for the zero rows that pad the last chunk: their v is zero, so they add nothing.
        u32x4 x = __builtin_bit_cast(u32x4, ak);
#pragma unroll
        for (int d = 0; d < 4; ++d) x[d] = (x[d] & t8_keep) | t8_const;
        ak = __builtin_bit_cast(bf16x8, x);
      }
      return ak;
    };
    auto unpack_k = [&](const bf16x8& kt) {
      const u32x4 x = __builtin_bit_cast(u32x4, kt);
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        k4[2 * d] = __builtin_bit_cast(float, x[d] << 16) * 0.25f;
        k4[2 * d + 1] = __builtin_bit_cast(float, x[d] & 0xFFFF0000u) * 0.25f;
      }
    };
    unpack_k(kt0);
    bf16x8 ak = psi_k(integral_constant<int, 0>{});
    if constexpr (kNorm) {
      K2 = mfma(kt0, kt0, K2);    // K2 += k^T k: the raw k^T tile is both operands (K2 is symmetric)
      K1 = mfma(kt0, ones8, K1);  // K1 += k^T 1
    }
    BASED_STAGE_END();

    // One slab of 32 tokens at a time; stage (s, i) runs the four MFMAs of slot tile i while the
    // operand of the next tile is generated and the finished tile before it is published.
    bf16x8 kt1 = load_kt(slot, kt_lane, 1);
    const bool more1 = t0 + kChunk < t_end;
    static_for<2 * kOwn>([&](auto ST) {
      constexpr int st = decltype(ST)::value;
      constexpr int s = st / kOwn, i = st % kOwn;
      if constexpr (s == 0 && i == kOwn - 1) {
#pragma unroll
        for (int et = 0; et < CTL; ++et) vt_s1[et] = load_vt(slot, vt_lane, vt_j, et, 1);
      }
#pragma unroll
      for (int et = 0; et < CTL; ++et) S[i][et] = mfma(ak, s == 0 ? vt_s0[et] : vt_s1[et], S[i][et]);
      if constexpr (st + 1 < 2 * kOwn) {
        if constexpr (i + 1 == kOwn) {  // the next stage starts slab 1
          unpack_k(kt1);
          if constexpr (kNorm) {
            K2 = mfma(kt1, kt1, K2);
            K1 = mfma(kt1, ones8, K1);
          }
        }
        ak = psi_k(integral_constant<int, (i + 1) % kOwn>{});
      }
      if constexpr (MODE != kModeDelta && s == 1 && i == 2) {
        if (more1) publish_pair(buf ^ 1);  // both tiles of the slab are final
      }
      interleave<CTL, (((i + 1 == kOwn && s == 0) ? 7 : (s == 1 && i == 2) ? 6 : 3) * 4 + CTL - 1) / CTL>();
      BASED_STAGE_END();
    });
    // the rest of the state after this chunk, for the next chunk's readers
    if constexpr (MODE != kModeDelta) {
      if (more1) {
        if constexpr (kOwn == 2) publish_pair(buf ^ 1);
        publish_single(buf ^ 1);
        publish_norm(buf ^ 1);
      }
    }
    // The next chunk's rows (requested one chunk ago) must have landed before anyone reads them;
    // the loads requested in this iteration may stay in flight if they were a whole chunk's.
    if (t0 + 3 * kChunk <= t_end) {
      barrier_updater<kInFlight>();
    } else {
      barrier_updater<0>();
    }
  }

  // ---------------- a segment's contribution goes to the workspace as it sits in registers ----------------
  if constexpr (MODE == kModeDelta) {
#pragma unroll
    for (int i = 0; i < kOwn; ++i)
#pragma unroll
      for (int et = 0; et < CT; ++et)
        *reinterpret_cast<f32x4*>(ws_mine + ws_tile(own_tile(w, i), et)) = S[i][et];
    if constexpr (kNorm) {
      // (every block's entry gets the normaliser state, so that the prefix pass reads nothing
      // that was never written; the workgroup takes it from its first block's entry)
#pragma unroll
      for (int blk = 0; blk < CT / 4; ++blk) {
        *reinterpret_cast<f32x4*>(ws_mine + blk * ws_block + kWsK2 + lane * 4) = K2;
        *reinterpret_cast<f32x4*>(ws_mine + blk * ws_block + kWsK1 + lane * 4) = K1;
      }
    }
    return;
  }

  // ---------------- expand the 160-slot state into the (dv, 273) decode layout ----------------
  // Sixteen channels at a time: the four updaters scatter their slot tiles of one channel
  // tile into a 16 x 273 fp32 block in LDS (each cross slot lands on both (i, j) and (j, i),
  // with the factor that undoes the packing weights), and the block, which is contiguous in
  // the decode state, leaves with coalesced 16-byte stores by the whole workgroup.
  if (kv_state != nullptr && last_seg) {
    float* blk = reinterpret_cast<float*>(lds + LD::kOffImg);
    static_assert(16 * kExp * 4 <= LD::kImgBytes, "expansion block must fit in a state image buffer");
    static_for<CTL>([&](auto ET) {
      constexpr int et = decltype(ET)::value;
      if (16 * et >= live_ch) return;  // uniform over the workgroup (the readers count the same rounds)
      __syncthreads();  // the buffer is free (main loop done / previous block copied out)
      float* row = blk + col * kExp;
      static_for<kOwn>([&](auto II) {
        constexpr int i = decltype(II)::value;
        constexpr int t = own_tile(w, i);
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
              row[0] = x;  // constant feature
            }
          } else {
            row[1 + j] = x * 2.0f;
          }
        }
      });
      __syncthreads();
      f32x4* dst = reinterpret_cast<f32x4*>(kv_state + (bh * dv + 64 * eb + 16 * et) * kExp);
      const f32x4* src = reinterpret_cast<const f32x4*>(blk);
      for (int idx = threadIdx.x; idx < 16 * kExp / 4; idx += kThreads) dst[idx] = src[idx];
    });
    // normaliser state = sum of phi(k): the token count, K1/2 and K2/(4 sqrt 2), straight from fp32
    if constexpr (kNorm) {
      if (eb == 0) {
        float* ks = k_state + bh * kExp;
        if (lane == 0) ks[0] = (float)L;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (col == 0) ks[1 + 4 * grp + r] = K1[r] * 0.5f;
          ks[1 + kFeat + 16 * (4 * grp + r) + col] = K2[r] * (0.25f / kSqrt2);
        }
      }
    }
  }
}
#undef BASED_STAGE_END

template <int MODE, int CT, int CTL = CT>
__global__ __launch_bounds__(kThreads, CT == 4 ? 4 : 2) void lin_prefill_mfma_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ k, const __bf16* __restrict__ v,
    __bf16* __restrict__ y, float* __restrict__ kv_state, float* __restrict__ k_state, int H, int L,
    int dv, long q_sb, long q_sh, long q_sl, long k_sb, long k_sh, long k_sl, long v_sb, long v_sh,
    long v_sl, long y_sb, long y_sh, long y_sl, float eps, float* __restrict__ ws, int seg_tokens, int n_seg) {
  __shared__ __align__(16) unsigned char lds[PrefillLds<CT>::kBytes];
#define BASED_CHAIN_ARGS lds, q, k, v, y, kv_state, k_state, H, L, dv, q_sb, q_sh, q_sl, k_sb, k_sh, \
                         k_sl, v_sb, v_sh, v_sl, y_sb, y_sh, y_sl, eps, ws, seg_tokens, n_seg
  switch (__builtin_amdgcn_readfirstlane(threadIdx.x >> 6)) {
    case 0: lin_prefill_reader<0, MODE, CT, CTL>(BASED_CHAIN_ARGS); break;
    case 1: lin_prefill_reader<1, MODE, CT, CTL>(BASED_CHAIN_ARGS); break;
    case 2: lin_prefill_reader<2, MODE, CT, CTL>(BASED_CHAIN_ARGS); break;
    case 3: lin_prefill_reader<3, MODE, CT, CTL>(BASED_CHAIN_ARGS); break;
    case 4: lin_prefill_updater<0, MODE, CT, CTL>(BASED_CHAIN_ARGS); break;
    case 5: lin_prefill_updater<1, MODE, CT, CTL>(BASED_CHAIN_ARGS); break;
    case 6: lin_prefill_updater<2, MODE, CT, CTL>(BASED_CHAIN_ARGS); break;
    default: lin_prefill_updater<3, MODE, CT, CTL>(BASED_CHAIN_ARGS); break;
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

// Head dims the MFMA kernel serves: whole 16-channel tiles.  A block of 64 channels per workgroup;
// the last block of a head dim that is no multiple of 64 (112 = 64 + 48, the released 1B / 1.3B
// models) runs with its missing tiles fed stand-in data and dropped at the stores.
static bool prefill_mfma_takes(int64_t dv) { return dv >= 16 && dv <= 1024 && dv % 16 == 0; }
// Head dims of 65..128 channels go to workgroups that carry both blocks of 64 (psi(q) and psi(k)
// generated once per head instead of once per block).
static bool prefill_wide(int64_t dv) { return dv > 64 && dv <= 128; }
// head dims 97..112 (the released 1B / 1.3B models have 112): seven live channel tiles in the wide workgroup
static bool prefill_live7(int64_t dv) { return dv > 96 && dv <= 112; }
// workgroups per (batch, head)
static int64_t prefill_workgroups_per_head(int64_t dv) { return prefill_wide(dv) ? 1 : (dv + 63) / 64; }

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
  if (io_dtype == BASED_BF16 && prefill_mfma_takes(dv)) {
    const int64_t strides[] = {q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, y_sb, y_sh, y_sl};
    for (int64_t st : strides)
      BASED_REQUIRE(st % 8 == 0, BASED_ERR_ALIGN,
                    "linear_attn_prefill: bf16 strides must be multiples of 8 elements (16 bytes)");
    BASED_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(y), BASED_ERR_ALIGN,
                  "linear_attn_prefill: tensors must be 16-byte aligned");
    BASED_REQUIRE(B * H * ((dv + 63) / 64) < (1ll << 31), BASED_ERR_SHAPE, "linear_attn_prefill: sizes too large");
    dim3 grid((unsigned)(B * H * prefill_workgroups_per_head(dv))), block(kThreads);
    auto kern = prefill_live7(dv) ? lin_prefill_mfma_kernel<kModeFull, 8, 7>
                : prefill_wide(dv) ? lin_prefill_mfma_kernel<kModeFull, 8> : lin_prefill_mfma_kernel<kModeFull, 4>;
    hipLaunchKernelGGL(kern, grid, block, 0, s, (const __bf16*)q, (const __bf16*)k,
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

// Workgroup slots of one full wave of the MFMA prefill kernel on MI355X (256 CUs x 2 resident
// workgroups); segment counts are chosen to fill about one such wave.
static constexpr int64_t kPrefillSlots = 512;
// Up to this many segments the second pass sums the earlier ones itself (measured: B=2, L=4096 as
// 8 segments 32.0 -> 28.7 us, B=1 as 16 segments 24.9 -> 23.9 us without the prefix launch; the
// planned segment counts beyond it belong to long sequences)
static constexpr int64_t kFoldSegments = 16;

extern "C" BASED_API int based_linear_attn_prefill_plan(int64_t B, int64_t H, int64_t L, int64_t dv,
                                                        int io_dtype, int64_t* n_seg,
                                                        int64_t* workspace_bytes) {
  using namespace based;
  BASED_REQUIRE(n_seg && workspace_bytes, BASED_ERR_ARG, "linear_attn_prefill_plan: null output pointer");
  *n_seg = 1;
  *workspace_bytes = 0;
  if (io_dtype != BASED_BF16 || !based::prefill_mfma_takes(dv) || B <= 0 || H <= 0 || L <= 0) return BASED_OK;
  const int64_t chains = B * H * ((dv + 63) / 64);
  const int64_t chunks = (L + kChunk - 1) / kChunk;
  // Measured on MI355X at L = 4096 (best segment count per batch size): 16 chains -> 16, 32 -> 8,
  // 48..128 -> 4, and from 192 chains on the single pass wins (one workgroup alone on a compute
  // unit is only 12 % slower per chunk than two sharing it, so filling the second slot does not
  // pay for the second pass over k and v).  Hence: about one workgroup per compute unit, at least
  // four segments (up to kFoldSegments need no prefix launch), and for long sequences segments of at most
  // 32 chunks while that still fits the resident slots.
  if (chains > kPrefillSlots / 4 || chunks < 2) return BASED_OK;
  int64_t want = chains <= 16 ? 16 : (chains <= 32 ? 8 : 4);
  while (want * 32 < chunks && chains * want * 2 <= kPrefillSlots) want *= 2;
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
  BASED_REQUIRE(io_dtype == BASED_BF16 && prefill_mfma_takes(dv), BASED_ERR_SHAPE,
                "%s: only the bf16 MFMA path (head dims that are multiples of 16) can be split", who);
  BASED_REQUIRE(B > 0 && H > 0 && L > 0 && B * H < (1ll << 31) && L < (1ll << 31), BASED_ERR_ARG, "%s: bad sizes", who);
  const int64_t chunks = (L + kChunk - 1) / kChunk;
  BASED_REQUIRE(n_seg >= 2 && n_seg <= chunks && n_seg < 65536, BASED_ERR_ARG, "%s: %ld segments for %ld chunks", who,
                (long)n_seg, (long)chunks);
  const int64_t seg_chunks = (chunks + n_seg - 1) / n_seg;
  BASED_REQUIRE((n_seg - 1) * seg_chunks < chunks, BASED_ERR_ARG,
                "%s: segment count %ld leaves empty segments (use the plan)", who, (long)n_seg);
  const int64_t eblocks = (dv + 63) / 64;
  const int64_t chains = B * H * eblocks;
  BASED_REQUIRE(chains < (1ll << 31), BASED_ERR_SHAPE, "%s: sizes too large", who);
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
  dim3 block(kThreads);
  // pass 1: every segment but the last accumulates its own contribution to the state
  const bool wide = prefill_wide(dv);
  const unsigned wgs = (unsigned)(B * H * prefill_workgroups_per_head(dv));  // a wide workgroup carries two chains
  const bool live7 = prefill_live7(dv);
  auto kern_delta = live7 ? lin_prefill_mfma_kernel<kModeDelta, 8, 7>
                    : wide ? lin_prefill_mfma_kernel<kModeDelta, 8> : lin_prefill_mfma_kernel<kModeDelta, 4>;
  hipLaunchKernelGGL(kern_delta, dim3(wgs, 1, (unsigned)(n_seg - 1)),
                     block, 0, s, (const __bf16*)q, (const __bf16*)k, (const __bf16*)v, (__bf16*)y, kv_state,
                     k_state, (int)H, (int)L, (int)dv, q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, y_sb,
                     y_sh, y_sl, eps, ws, seg_tokens, (int)n_seg);
  int rc = check_launch(who);
  if (rc) return rc;
  // With up to kFoldSegments segments every workgroup of the second pass adds up the contributions
  // before its own (reads of 42 KB each, mostly from L2: cheaper than one more launch); with more,
  // a prefix pass over the workspace is cheaper than every workgroup reading half of its chain's
  // entries.
  const bool fold = n_seg <= kFoldSegments;
  if (!fold) {
    hipLaunchKernelGGL(lin_prefill_prefix_kernel, dim3((unsigned)chains, (kSegStateFloats / 4 + 255) / 256), dim3(256), 0,
                       s, ws, (int)n_seg);
    rc = check_launch(who);
    if (rc) return rc;
  }
  auto kern_from = fold ? (live7 ? lin_prefill_mfma_kernel<kModeFromSum, 8, 7>
                           : wide ? lin_prefill_mfma_kernel<kModeFromSum, 8> : lin_prefill_mfma_kernel<kModeFromSum, 4>)
                        : (live7 ? lin_prefill_mfma_kernel<kModeFrom, 8, 7>
                           : wide ? lin_prefill_mfma_kernel<kModeFrom, 8> : lin_prefill_mfma_kernel<kModeFrom, 4>);
  hipLaunchKernelGGL(kern_from, dim3(wgs, 1, (unsigned)n_seg),
                     block, 0, s, (const __bf16*)q, (const __bf16*)k, (const __bf16*)v, (__bf16*)y, kv_state,
                     k_state, (int)H, (int)L, (int)dv, q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, y_sb,
                     y_sh, y_sl, eps, ws, seg_tokens, (int)n_seg);
  return check_launch(who);
}

// Scratch of based_linear_attn_prefill_split_static: one array per GPU, part of the code object,
// alive until the process ends.  64 MiB hold 1560 (chain, segment) state images of 43,008 bytes,
// more than any plan the plan entry point returns (it fills at most kPrefillSlots = 512 workgroup
// slots, i.e. at most 512 images).  In host code the array's name is only a handle for
// hipGetSymbolAddress; the device address is looked up once per device and kept in g_scratch_ptr.
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
  // Size check first: an oversized request is refused without touching the device.  Every factor
  // is bounded before the product is formed (B * H < 2^31, at most 2 channel blocks, n_seg < 2^16,
  // 43,008 bytes per image: below 2^63).
  BASED_REQUIRE(B > 0 && H > 0 && B < (1ll << 31) && H < (1ll << 31) && B * H < (1ll << 31) && n_seg < 65536 &&
                    L > 0 && L < (1ll << 31),
                BASED_ERR_ARG, "linear_attn_prefill_split_static: bad sizes");
  if (io_dtype == BASED_BF16 && prefill_mfma_takes(dv)) {
    const int64_t chains = B * H * ((dv + 63) / 64);
    BASED_REQUIRE(chains * n_seg * (int64_t)kSegStateFloats * 4 <= kStaticScratchBytes, BASED_ERR_SHAPE,
                  "linear_attn_prefill_split_static: %ld chains x %ld segments need %ld bytes of scratch, the "
                  "static array holds %ld",
                  (long)chains, (long)n_seg, (long)(chains * n_seg * (int64_t)kSegStateFloats * 4),
                  (long)kStaticScratchBytes);
  }
  void* scratch = static_scratch_for_current_device("linear_attn_prefill_split_static");
  if (scratch == nullptr) return BASED_ERR_LAUNCH;
  return launch_prefill_split("linear_attn_prefill_split_static", q, k, v, y, kv_state, k_state, B, H, L, dv, q_sb,
                              q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, y_sb, y_sh, y_sl, eps, io_dtype, n_seg,
                              scratch, kStaticScratchBytes, kStaticScratchBytes, stream);
}
