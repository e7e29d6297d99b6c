// Sliding-window causal softmax attention for gfx950: prefill (MFMA) and decode step.
//
// Prefill.  Four wavefronts cover 64 consecutive queries of one (batch, head); wavefront w owns
// queries [q0+16w, q0+16w+16) and the keys [n0-64(NB-1), n0+16) they can see: NB = 2 staged
// blocks of 64 rows for a window of up to 64 to the left (80 keys, 5 tiles), NB = 3 for up to 128
// (144 keys, 9 tiles), plus the causal diagonal.
//   S^T = K Q^T   : 5 or 9 key tiles x 2 MFMA 16x16x32 (head dim 64); the K rows are staged once
//                   in LDS (a lane's operand = 8 consecutive bf16 of one row).
//   softmax       : S^T leaves the MFMA with lane <-> query and registers <-> keys, so the
//                   row max / row sum are in-lane loops plus two cross-lane steps.
//   O^T = V^T P^T : the accumulator layout of S^T is already the B-operand layout for a
//                   product contracted over keys, so P never leaves registers.  V^T (lane
//                   <-> channel, registers <-> keys) is the one operand that needs a
//                   transpose: V rows are staged as they come and read with the transposing
//                   LDS load.  The 16 x 64 output tile of a wavefront is staged in 16 LDS rows
//                   that are its own at that moment, so that every lane stores 16 bytes of a
//                   full 128-byte row.
// Whole-window softmax in one pass: 80 (144) keys fit in registers, so no online rescaling.
// A workgroup holds G such wavefront quartets, one per head of G heads that are neighbours in
// memory (G = 4 or 2 when the head stride is 64 elements; the launcher says which): their rows of
// one token are one contiguous 128 G-byte piece, and HBM serves longer pieces measurably better
// (a plain streaming kernel with this access pattern: 4.5 TB/s at 128 bytes, 5.1 at 256, 5.3 at
// 512).
// LDS rows are 128 bytes, unpadded; the 16-byte pieces of a row are XOR-swizzled by the row
// number so that the operand reads (16 rows x 16 bytes, or 8 rows x 32 bytes for the transposing
// read) fall on distinct banks.
//
// Decode.  One workgroup of four wavefronts per (batch, head) against the last w_left+1 rows of
// a linear cache, with every load issued up front (one memory round trip per step).
#include "common.hpp"

#include <atomic>

namespace based {

constexpr int kHeadDim = 64;
constexpr int kQTile = 64;          // queries per wavefront quartet
constexpr int kRowBytes = 128;      // a K, V or Q row in LDS

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// 16-byte piece p (0..7) of LDS row r sits at piece p ^ swizzle(r).
//   K and Q rows are read as MFMA operands, 16 consecutive rows x one piece each: rows r and r+1
//   differ in the bank half (128-byte rows), rows of the same parity need 8 different pieces.
//   V rows are read by the transposing load, 8 consecutive rows x two neighbouring pieces each:
//   rows of the same parity need 4 different piece pairs.
__device__ __forceinline__ int swz_k(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int swz_v(int row) { return ((row >> 1) & 3) << 1; }

// bf16 pair (x1 at channel c < 32, x2 at channel c + 32) -> rotated pair, rounded to bf16
__device__ __forceinline__ void rope_rotate8(u32x4& lo, u32x4& hi, const f32x4 (&cs)[2], const f32x4 (&sn)[2]) {
  u32x4 out_lo, out_hi;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    float o1[2], o2[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int j = 2 * d + e;
      const float x1 = bf16_bits_to_f32(e == 0 ? (lo[d] & 0xFFFFu) : (lo[d] >> 16));
      const float x2 = bf16_bits_to_f32(e == 0 ? (hi[d] & 0xFFFFu) : (hi[d] >> 16));
      const float c = cs[j >> 2][j & 3], sgn = sn[j >> 2][j & 3];
      o1[e] = x1 * c - x2 * sgn;
      o2[e] = x1 * sgn + x2 * c;
    }
    out_lo[d] = pack_bf16(o1[0], o1[1]);
    out_hi[d] = pack_bf16(o2[0], o2[1]);
  }
  lo = out_lo;
  hi = out_hi;
}

// One tile's worth of rows on their way from global memory to LDS (register prefetch).
struct SwaRows {
  u32x4 kp[2], vp[2], qp[2];  // qp: only when the queries go through LDS
  f32x4 cs[2], sn[2];         // rotary factors (ROPE only)
};

// per head: the K and V rings, and with paired heads 64 query rows (see QLDS in the kernel)
constexpr int swa_head_lds_bytes(int nb, int g) { return (2 * nb + (g > 1 ? 1 : 0)) * kQTile * kRowBytes; }

// ROPE: q and k are rotated on their way into LDS (non-interleaved rotary over the whole head,
// cos/sin tables of 32 frequencies per position), as flash-attn's rotary layer does before the
// attention of the reference (slide_attention.py:346-355,553-556).
// kc_out / vc_out (optional): the (rotated) K rows and the V rows of this call are also written
// to a KV cache, the job of _update_kv_cache (slide_attention.py:255-281).
// G > 1 needs q_sh == k_sh == v_sh == o_sh == c_sh == 64 and H % G == 0 (checked by the launcher).
template <bool ROPE, int NB, int G>
__global__ __launch_bounds__(256 * G, G >= 2 ? (NB == 3 ? 2 : 4) : (NB == 3 || ROPE ? 3 : 4)) void swa_prefill_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ k, const __bf16* __restrict__ v,
    __bf16* __restrict__ o, int H, int L, int n_tiles, int run_tiles, long q_sb, long q_sl, long q_sh,
    long k_sb, long k_sl, long k_sh, long v_sb, long v_sl, long v_sh, long o_sb, long o_sl, long o_sh,
    int w_left, float scale_log2e, const float* __restrict__ rope_cos, const float* __restrict__ rope_sin,
    __bf16* __restrict__ kc_out, __bf16* __restrict__ vc_out, long c_sb, long c_st, long c_sh) {
  // Per head: a ring of NB blocks of 64 K rows, the same of V rows, and (ROPE) the 64 rotated
  // queries.  One block holds the current tile's own keys, the others the 64 (NB - 1) keys to its
  // left.  Moving on by one tile, "own" becomes "left" without a copy and the oldest block takes
  // the next tile's rows.
  constexpr int NT = 4 * (NB - 1) + 1;   // key tiles of 16 a wavefront sees
  constexpr int NS = (NT + 1) / 2;       // key slabs of 32 in the second product (last one half empty)
  // Where the queries and the finished output tile pass through:
  //   paired heads (QLDS): queries are fetched with the K rows (256-byte pieces) into 64 LDS rows
  //     of their own; a wavefront's 16 of them, free once its operand is in registers, later stage
  //     its output tile.
  //   one head: every lane fetches its own operand from global memory one tile ahead (and rotates
  //     it in registers: the channel pairs c, c + 32 of the rotation are the same lane's two operand
  //     halves); the output tile is staged in the wavefront's 16 rows of the oldest K block, which
  //     only this wavefront rewrites.  No LDS beyond the rings: 48 KB for the three-block ring,
  //     three workgroups per compute unit.
  constexpr bool QLDS = G > 1;
  constexpr int kHeadBytes = swa_head_lds_bytes(NB, G);
  constexpr int kOffV = NB * kQTile * kRowBytes;
  constexpr int kOffQ = 2 * kOffV;
  extern __shared__ __align__(16) unsigned char swa_lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wq = wave & 3;     // which 16 of the tile's 64 queries
  const int hsel = wave >> 2;  // which of the workgroup's G heads
  const int col = lane & 15;   // query (B operand / accumulator column), or row of an A tile
  const int grp = lane >> 4;   // 0..3: which 8 contraction slots / which 4 accumulator rows

  // work item: a run of up to run_tiles consecutive query tiles of G neighbouring heads of one batch entry
  const int runs_per_seq = (n_tiles + run_tiles - 1) / run_tiles;
  // Order of the work items over the workgroup ids, by measurement (alternating runs on one box,
  // B=8, L=4096, cold).  Paired heads without the rotary: the head groups of one run of tokens are
  // neighbours; they read neighbouring 256-byte pieces of the same rows at about the same time
  // (59.7 -> 58.0 us).  With the rotary (65.7 against 68.6 us; with the cache fill as well the two
  // orders are equal) and with one head per workgroup (the other order is 2 % slower, 7 % with
  // rotary and cache fill): the runs of one head group are neighbours.
  // Runs in both directions (paired heads, two-block ring, no rotary, no cache fill): the first
  // tile of a run needs the 64 keys before it, which are the last tile's own keys of the run
  // before.  Even runs walk their tiles downwards, odd runs upwards, and all runs of a head group
  // sit behind one L2 (workgroup ids 8 apart): run 2m starts with its last tile at the moment
  // run 2m + 1 fetches that tile's keys as its halo, and run 2m + 1 ends with its last tile when
  // run 2m + 2, coming down, needs it: the second fetch of those rows is served by the L2
  // (B=8, H=16, L=4096, 64 keys to the left: 216.1 -> 201.5 MB fetched per launch, which is q, k
  // and v once; 54.0 -> 53.3 us).  The results do not depend on the direction.
  constexpr bool kBidir = !ROPE && G > 1 && NB == 2;
  const int n_hg = gridDim.x / runs_per_seq;  // head groups of the whole batch
  const bool bidir = kBidir && kc_out == nullptr && runs_per_seq > 1 && n_hg % 8 == 0;
  int hg, run, b;
  if (bidir) {
    const int bhg = (int)(blockIdx.x % (unsigned)n_hg);
    run = (int)(blockIdx.x / (unsigned)n_hg);
    hg = bhg % (H / G), b = bhg / (H / G);
  } else if constexpr (G > 1 && !ROPE) {
    hg = (int)(blockIdx.x % (unsigned)(H / G));
    const unsigned rest = blockIdx.x / (unsigned)(H / G);
    run = (int)(rest % (unsigned)runs_per_seq), b = (int)(rest / (unsigned)runs_per_seq);
  } else {
    run = (int)(blockIdx.x % (unsigned)runs_per_seq);
    const unsigned bhg = blockIdx.x / (unsigned)runs_per_seq;
    hg = (int)(bhg % (unsigned)(H / G)), b = (int)(bhg / (unsigned)(H / G));
  }
  const int tile_begin = run * run_tiles;
  const int tile_end = tile_begin + run_tiles < n_tiles ? tile_begin + run_tiles : n_tiles;
  const bool down = bidir && (run & 1) == 0;
  // from one tile to the next: the queries move by q_step; the rows fetched are the next tile's
  // own (upwards) or the block of keys at the far left of its window (downwards), q_ahead tokens
  // before its queries
  const int q_step = down ? -kQTile : kQTile;
  const int q_ahead = down ? kQTile * (NB - 1) : 0;

  // rows are moved by lane-dependent heads (head0 + mv_head); the products are per wavefront (head0 + hsel)
  const long head0 = (long)hg * G;
  unsigned char* const my = swa_lds + hsel * kHeadBytes;

  // Pieces (row of a 64-row block, 16-byte piece, head) moved by this thread.  The G wavefronts
  // with the same wq move the rows 16 wq .. 16 wq + 15 of all G heads between them, every load
  // instruction covering whole 128 G-byte pieces of memory.
  //   plain: instruction i of 2 moves 8/G rows x G heads x 8 pieces
  //   ROPE : one row per 4 G lanes, pieces p and p + 4 (the channel pairs of the rotation)
  // V rows are never rotated: with the three-block ring they move in the plain arrangement (whole
  // rows per load and per cache store) also in the ROPE variant (rotary + cache fill at 128 keys
  // to the left 99.0 -> 94.8 us); with the two-block ring they follow K's arrangement (the plain
  // one measures 1 % slower there).
  constexpr bool kPlainV = !ROPE || NB == 3;
  const int mv_head = ROPE ? (lane >> 2) % G : (lane >> 3) % G;
  const int mv_head_v = kPlainV ? (lane >> 3) % G : mv_head;
  auto piece_row = [&](int i) {
    return ROPE ? 16 * wq + (16 / G) * hsel + lane / (4 * G) : 16 * wq + (16 / G) * hsel + (8 / G) * i + lane / (8 * G);
  };
  auto piece_idx = [&](int i) { return ROPE ? (lane & 3) + 4 * i : (lane & 7); };
  auto piece_row_v = [&](int i) {
    return kPlainV ? 16 * wq + (16 / G) * hsel + (8 / G) * i + lane / (8 * G) : piece_row(i);
  };
  auto piece_idx_v = [&](int i) { return kPlainV ? (lane & 7) : piece_idx(i); };
  const __bf16* const q_mv = q + b * q_sb + (head0 + mv_head) * q_sh;
  const __bf16* const k_mv = k + b * k_sb + (head0 + mv_head) * k_sh;
  const __bf16* const v_mv = v + b * v_sb + (head0 + mv_head_v) * v_sh;
  __bf16* kc_mv = nullptr;
  __bf16* vc_mv = nullptr;
  if (kc_out != nullptr) {
    kc_mv = kc_out + b * c_sb + (head0 + mv_head) * c_sh;
    vc_mv = vc_out + b * c_sb + (head0 + mv_head_v) * c_sh;
  }
  unsigned char* const mv_lds = swa_lds + mv_head * kHeadBytes;
  unsigned char* const mv_lds_v = swa_lds + mv_head_v * kHeadBytes;
  __bf16* const o_my = o + b * o_sb + (head0 + hsel) * o_sh;

  // No load sits under a condition (a load in a branch is waited for at the end of the branch,
  // which would also end any overlap with the arithmetic): rows outside the sequence are fetched
  // from its nearest row instead.  Keys before the start are masked, keys and queries past the end
  // belong to rows that are never stored, so what is fetched for them does not matter.
  auto load_rows = [&](int key0, SwaRows& r, bool with_q, int q_off = 0) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      int key = key0 + piece_row(i);
      int qrow = key + q_off;
      qrow = qrow < 0 ? 0 : (qrow < L ? qrow : L - 1);
      key = key < 0 ? 0 : (key < L ? key : L - 1);
      r.kp[i] = *reinterpret_cast<const u32x4*>(k_mv + (long)key * k_sl + 8 * piece_idx(i));
      int key_v = key0 + piece_row_v(i);
      key_v = key_v < 0 ? 0 : (key_v < L ? key_v : L - 1);
      r.vp[i] = *reinterpret_cast<const u32x4*>(v_mv + (long)key_v * v_sl + 8 * piece_idx_v(i));
      if constexpr (QLDS)
        if (with_q) r.qp[i] = *reinterpret_cast<const u32x4*>(q_mv + (long)qrow * q_sl + 8 * piece_idx(i));  // a literal at every call
    }
    if constexpr (ROPE) {
      int key = key0 + piece_row(0);
      key = key < 0 ? 0 : (key < L ? key : L - 1);
      const f32x4* c4 = reinterpret_cast<const f32x4*>(rope_cos + (long)key * (kHeadDim / 2) + 8 * (lane & 3));
      const f32x4* s4 = reinterpret_cast<const f32x4*>(rope_sin + (long)key * (kHeadDim / 2) + 8 * (lane & 3));
      r.cs[0] = c4[0];
      r.cs[1] = c4[1];
      r.sn[0] = s4[0];
      r.sn[1] = s4[1];
    }
  };
  // own_rows: the rows are the tile's own keys (they also carry its queries and go to the cache)
  auto store_rows = [&](int blk, int key0, SwaRows& r, bool own_rows) {
    if constexpr (ROPE) {
      rope_rotate8(r.kp[0], r.kp[1], r.cs, r.sn);
      if constexpr (QLDS)
        if (own_rows) rope_rotate8(r.qp[0], r.qp[1], r.cs, r.sn);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int lrow = piece_row(i);
      const int row = blk * kQTile + lrow;
      const int pc = piece_idx(i);
      const int lrow_v = piece_row_v(i);
      *reinterpret_cast<u32x4*>(mv_lds + row * kRowBytes + ((pc ^ swz_k(lrow)) << 4)) = r.kp[i];
      *reinterpret_cast<u32x4*>(mv_lds_v + kOffV + (blk * kQTile + lrow_v) * kRowBytes + ((piece_idx_v(i) ^ swz_v(lrow_v)) << 4)) = r.vp[i];
      if constexpr (QLDS)
        if (own_rows) *reinterpret_cast<u32x4*>(mv_lds + kOffQ + lrow * kRowBytes + ((pc ^ swz_k(lrow)) << 4)) = r.qp[i];
      // Cache rows leave non-temporally, an instruction writing whole rows: as they are in the
      // plain arrangement, after an exchange between lanes in the rotary one (below; half rows
      // from two instructions have to be merged by the cache, and non-temporal half rows were
      // slower still, 99 -> 103 us).
      const int key = key0 + lrow;
      if constexpr (!kPlainV) {
        // (both in the rotary arrangement: after the loop)
      } else if (own_rows && kc_mv != nullptr) {
        const int key_v = key0 + lrow_v;
        if constexpr (!ROPE) {
          if (key < L) __builtin_nontemporal_store(r.kp[i], reinterpret_cast<u32x4*>(kc_mv + (long)key * c_st + 8 * pc));
        }
        if (key_v < L)
          __builtin_nontemporal_store(r.vp[i], reinterpret_cast<u32x4*>(vc_mv + (long)key_v * c_st + 8 * piece_idx_v(i)));
      }
    }
    if constexpr (ROPE) {
      // Rotated K rows for the cache (and, where V moves in the rotary arrangement too, the V rows).  In the rotary arrangement four lanes hold a row (lane q:
      // pieces q and q + 4), so a store instruction would write half rows.  Neighbouring groups of
      // four (the next head, or with one head per workgroup the next row) swap halves first
      // (lower group gives its pieces 4..7, upper group its pieces 0..3, through a mirror of the
      // eight lanes): then eight lanes hold one whole row per register and both stores write whole
      // 128-byte rows, non-temporally like the V rows.
      if (own_rows && kc_mv != nullptr) {
        const bool upper = (lane >> 2) & 1;
        const int ql = lane & 3;
        u32x4 row_lo, row_hi;  // the lower group's row: pieces q | 7 - q; the upper group's: pieces 3 - q | q + 4
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const uint32_t give = upper ? r.kp[0][d] : r.kp[1][d];
          const uint32_t got = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)give, 0x141 /* row_half_mirror */, 0xf, 0xf, false);
          row_lo[d] = upper ? got : r.kp[0][d];
          row_hi[d] = upper ? r.kp[1][d] : got;
        }
        const int key = key0 + piece_row(0);
        __bf16* base_lo = kc_mv;
        __bf16* base_hi = kc_mv;
        int key_lo = key, key_hi = key;
        if constexpr (G >= 2) {
          base_lo = upper ? kc_mv - c_sh : kc_mv;
          base_hi = upper ? kc_mv : kc_mv + c_sh;
        } else {
          key_lo = upper ? key - 1 : key;
          key_hi = upper ? key : key + 1;
        }
        const int piece_lo = upper ? 7 - ql : ql, piece_hi = upper ? ql + 4 : 3 - ql;
        if (key_lo < L) __builtin_nontemporal_store(row_lo, reinterpret_cast<u32x4*>(base_lo + (long)key_lo * c_st + 8 * piece_lo));
        if (key_hi < L) __builtin_nontemporal_store(row_hi, reinterpret_cast<u32x4*>(base_hi + (long)key_hi * c_st + 8 * piece_hi));
        if constexpr (!kPlainV) {
          u32x4 v_lo, v_hi;
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            const uint32_t give = upper ? r.vp[0][d] : r.vp[1][d];
            const uint32_t got = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)give, 0x141, 0xf, 0xf, false);
            v_lo[d] = upper ? got : r.vp[0][d];
            v_hi[d] = upper ? r.vp[1][d] : got;
          }
          const long k_to_v = vc_mv - kc_mv;  // the V rows of the cache lie at a fixed distance from the K rows
          if (key_lo < L) __builtin_nontemporal_store(v_lo, reinterpret_cast<u32x4*>(base_lo + k_to_v + (long)key_lo * c_st + 8 * piece_lo));
          if (key_hi < L) __builtin_nontemporal_store(v_hi, reinterpret_cast<u32x4*>(base_hi + k_to_v + (long)key_hi * c_st + 8 * piece_hi));
        }
      }
    }
  };
  // one head per workgroup: the Q operand of this lane's query (channels 32 ds + 8 grp ..+7),
  // rotated in place when ROPE
  const __bf16* const q_my = q + b * q_sb + (head0 + hsel) * q_sh;
  auto load_q = [&](int q0, bf16x8 (&bq)[2]) {
    int n = q0 + 16 * wq + col;
    n = n < L ? n : L - 1;  // queries past the end are never stored
    u32x4 x[2];
#pragma unroll
    for (int ds = 0; ds < 2; ++ds) x[ds] = *reinterpret_cast<const u32x4*>(q_my + (long)n * q_sl + 32 * ds + 8 * grp);
    if constexpr (ROPE) {
      f32x4 cs[2], sn[2];
      const f32x4* c4 = reinterpret_cast<const f32x4*>(rope_cos + (long)n * (kHeadDim / 2) + 8 * grp);
      const f32x4* s4 = reinterpret_cast<const f32x4*>(rope_sin + (long)n * (kHeadDim / 2) + 8 * grp);
      cs[0] = c4[0];
      cs[1] = c4[1];
      sn[0] = s4[0];
      sn[1] = s4[1];
      rope_rotate8(x[0], x[1], cs, sn);
    }
    bq[0] = __builtin_bit_cast(bf16x8, x[0]);
    bq[1] = __builtin_bit_cast(bf16x8, x[1]);
  };

  int q0 = (down ? tile_end - 1 : tile_begin) * kQTile;
  SwaRows pre;
  bf16x8 bq[2], bq_next[2];
  {
    // first tile: own rows in block 0, the keys 64 a to the left in block NB - a (one round trip)
    SwaRows left[NB - 1];
#pragma unroll
    for (int a = 1; a < NB; ++a) load_rows(q0 - a * kQTile, left[a - 1], false);
    load_rows(q0, pre, true);
    if constexpr (!QLDS) load_q(q0, bq);
#pragma unroll
    for (int a = 1; a < NB; ++a) store_rows(NB - a, q0 - a * kQTile, left[a - 1], false);
    store_rows(0, q0, pre, true);
  }
  if (tile_begin + 1 < tile_end) {  // the next tile's rows travel while this one is computed
    load_rows(q0 + q_step - q_ahead, pre, true, q_ahead);
    if constexpr (!QLDS) load_q(q0 + kQTile, bq_next);
  }

  // lane-constant parts of the operand addresses (rows of a tile start at multiples of 16)
  const int k_lane = col * kRowBytes;                  // + ((4 ds + grp) ^ swz_k(col)) << 4
  const int k_sw = swz_k(col);
  const int vt_row = 4 * grp + (col >> 2);             // row of a 16-row tile this lane fetches for the transposing read
  const int v_lane = vt_row * kRowBytes + 8 * (col & 1);
  const int v_sw = swz_v(vt_row);
  const int v_half = (col & 3) >> 1;                   // piece 2 et + v_half

  // key tiles i < i_win reach below the window of the wavefront's last query (see the softmax)
  const int i_win = w_left >= 64 * (NB - 1) + 15 ? 0 : (64 * (NB - 1) + 30 - w_left) >> 4;
  // With 128 keys to the left the arithmetic, not the memory, sets the pace (144 keys per
  // wavefront and tile), a good part of it the addresses of the operand reads.  Paired heads there
  // run two wavefronts per SIMD and have registers to spare: their loop is unrolled over the three
  // positions of the ring, so that where a wavefront's tiles of 16 staged keys sit in LDS is, but
  // for the tiles whose wrap round the ring depends on the wavefront (their addresses wait in
  // registers), an immediate offset of the operand reads (B=8, H=16, L=4096, cold: rotary + cache
  // fill 95.0 -> 90.3 us; plain 63.8 -> 61.8 and rotary 78.4 -> 73.4 against one head per
  // workgroup).  The other variants lose what they gain to register spills, or have nothing to gain
  // because they wait for memory.
  constexpr bool kStaticRing = NB == 3 && G == 2;
  if constexpr (kStaticRing) {
    // a run starts with the own keys in block 0: the oldest block is 1, then 2, then 0
    for (int tile = tile_begin;;) {
      {
        constexpr int oldest = 1;
#include "swa_tile.inc"
      }
      q0 += kQTile;
      if (++tile == tile_end) break;
      {
        constexpr int oldest = 2;
#include "swa_tile.inc"
      }
      q0 += kQTile;
      if (++tile == tile_end) break;
      {
        constexpr int oldest = 0;
#include "swa_tile.inc"
      }
      q0 += kQTile;
      if (++tile == tile_end) break;
    }
  } else {
    int own = 0;  // ring block with keys [q0, q0+64); block own + 1 (mod NB) is the oldest
    for (int tile = tile_begin; tile < tile_end; ++tile, q0 += q_step) {
      const int oldest = own + 1 == NB ? 0 : own + 1;
#include "swa_tile.inc"
      // upwards the oldest block has taken the next tile's own rows; downwards the block of this
      // tile's own rows has taken the keys at the far left of the next tile's window
      own = down ? (own == 0 ? NB - 1 : own - 1) : oldest;
    }
  }
}

// One workgroup of four wavefronts per (b, h).  Keys lo..pos, lo = max(0, pos - w_left): at most
// 64 KB cached rows plus the new token (KB = 1 for windows of up to 64 to the left, 2 for up to
// 128).  Every global load of the step (K rows for the scores, V rows for the output) is issued
// before anything is waited on, so the step costs one memory round trip: thread t scores keys
// t/4 (+64) over channels 16 (t%4)..+16, and accumulates channel t%64 over the keys congruent to
// t/64 mod 4.
template <int KB>
__global__ __launch_bounds__(256) void swa_step_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ k_new, const __bf16* __restrict__ v_new,
    __bf16* __restrict__ kcache, __bf16* __restrict__ vcache, __bf16* __restrict__ o,
    const int32_t* __restrict__ cache_seqlens, int pos_host, int H, int max_seqlen, long q_sb,
    long q_sh, long kn_sb, long kn_sh, long vn_sb, long vn_sh, long o_sb, long o_sh, long c_sb,
    long c_st, long c_sh, int w_left, float scale_log2e, const float* __restrict__ rope_cos,
    const float* __restrict__ rope_sin, int rope_len) {
  constexpr int kCached = 64 * KB;   // most cached rows a step reads
  __shared__ float s_p[kCached + 16];  // scores, then weights; entry kCached is the new token
  __shared__ float s_part[4][kHeadDim];
  __shared__ __align__(16) float s_qrot[4][kHeadDim];  // rotated query, one private copy per wavefront
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bh = blockIdx.x;
  const int b = bh / H, h = bh % H;
  int pos = cache_seqlens ? cache_seqlens[b] : pos_host;
  pos = __builtin_amdgcn_readfirstlane(pos);
  if (pos < 0 || pos >= max_seqlen || (rope_cos != nullptr && pos >= rope_len)) {
    // A device-side position outside the cache or the rotary table cannot be reported to the
    // host from here (the call may be a graph replay): the cache is left untouched and the
    // output row of this (batch, head) is NaN, so the failure is visible downstream.
    if (wave == 0) o[b * o_sb + h * o_sh + lane] = (__bf16)__builtin_nanf("");
    return;
  }

  __bf16* kc = kcache + b * c_sb + h * c_sh;
  __bf16* vc = vcache + b * c_sb + h * c_sh;
  const int lo = pos - w_left > 0 ? pos - w_left : 0;
  const int ncached = pos - lo;  // 0..kCached rows of the cache, then the new token itself

  // ---- issue every load of the step ----
  const int kj = tid >> 2, kq4 = tid & 3;  // key (and key + 64) and channel quarter for the scores
  bf16x8 kx[KB][2];
#pragma unroll
  for (int g = 0; g < KB; ++g) {
    kx[g][0] = kx[g][1] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    if (kj + 64 * g < ncached) {
      const bf16x8* row = reinterpret_cast<const bf16x8*>(kc + (long)(lo + kj + 64 * g) * c_st + 16 * kq4);
      kx[g][0] = row[0];
      kx[g][1] = row[1];
    }
  }
  const bf16x8* qrow = reinterpret_cast<const bf16x8*>(q + b * q_sb + h * q_sh + 16 * kq4);
  const bf16x8 qx[2] = {qrow[0], qrow[1]};
  float cs = 1.0f, sn = 0.0f;  // rotary factors of channel `lane` at this position
  if (rope_cos != nullptr) {
    cs = rope_cos[(long)pos * (kHeadDim / 2) + (lane & 31)];
    sn = rope_sin[(long)pos * (kHeadDim / 2) + (lane & 31)];
  }
  constexpr int kPerWave = kCached / 4;  // keys of this wavefront: j = wave, wave + 4, ...
  // No load sits under a condition: a load in a branch is waited for at the end of the branch,
  // and these sixteen would be sixteen memory round trips one after the other.  Rows past the
  // window are fetched from row `lo` (inside the cache) and masked to zero as bits.
  float vv[kPerWave];
  const uint16_t* vc16 = reinterpret_cast<const uint16_t*>(vc);
#pragma unroll
  for (int u = 0; u < kPerWave; ++u) {
    const int j = 4 * u + wave;
    const bool in_window = j < ncached;
    const uint32_t raw = vc16[(long)(lo + (in_window ? j : 0)) * c_st + lane];
    vv[u] = bf16_bits_to_f32(raw & (in_window ? 0xffffu : 0u));
  }
  float kn = to_f32(k_new[b * kn_sb + h * kn_sh + lane]);
  const float vn = to_f32(v_new[b * vn_sb + h * vn_sh + lane]);
  float ql = to_f32(q[b * q_sb + h * q_sh + lane]);
  // this thread's slice of the query for the scores: 16 channels from 16 kq4
  float qf[16];
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int i = 0; i < 8; ++i) qf[8 * c + i] = to_f32(qx[c][i]);
  if (rope_cos != nullptr) {
    // Non-interleaved rotary over the whole head: channel c pairs with c +- 32,
    //   out[c] = x[c] cos - x[c+32] sin (c < 32),  out[c] = x[c] cos + x[c-32] sin (c >= 32),
    // rounded to bf16 like the rotated tensors of the prefill.  Every wavefront rotates the
    // query for itself (lane <-> channel) and hands the slices round through its own LDS row.
    const float sgn = lane < 32 ? -1.0f : 1.0f;
    ql = to_f32((__bf16)__builtin_fmaf(ql, cs, sgn * __shfl_xor(ql, 32, 64) * sn));
    kn = to_f32((__bf16)__builtin_fmaf(kn, cs, sgn * __shfl_xor(kn, 32, 64) * sn));
    s_qrot[wave][lane] = ql;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const f32x4* src = reinterpret_cast<const f32x4*>(&s_qrot[wave][16 * kq4]);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const f32x4 x = src[i];
      qf[4 * i + 0] = x[0];
      qf[4 * i + 1] = x[1];
      qf[4 * i + 2] = x[2];
      qf[4 * i + 3] = x[3];
    }
  }
  if (wave == 0) {  // the new token joins the cache (row pos)
    kc[(long)pos * c_st + lane] = (__bf16)kn;
    vc[(long)pos * c_st + lane] = (__bf16)vn;
  }

  // ---- scores ----
#pragma unroll
  for (int g = 0; g < KB; ++g) {
    float part = 0.f;
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int i = 0; i < 8; ++i) part = __builtin_fmaf(to_f32(kx[g][c][i]), qf[8 * c + i], part);
    part += __shfl_xor(part, 1, 64);
    part += __shfl_xor(part, 2, 64);
    if (kq4 == 0) s_p[kj + 64 * g] = kj + 64 * g < ncached ? part * scale_log2e : -INFINITY;
  }
  if (wave == 0) {
    const float self = wave_sum(ql * kn);
    if (lane == 0) s_p[kCached] = self * scale_log2e;
  }
  __syncthreads();

  // ---- softmax over the kCached + 1 entries (every wavefront redundantly: no second barrier) ----
  float sc[KB], pw[KB];
  const float s1 = s_p[kCached];
  float mx = s1;
#pragma unroll
  for (int g = 0; g < KB; ++g) {
    sc[g] = s_p[lane + 64 * g];
    mx = fmaxf(mx, sc[g]);
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, 64));
  const float p1 = __builtin_amdgcn_exp2f(s1 - mx);
  float psum = 0.f;
#pragma unroll
  for (int g = 0; g < KB; ++g) {
    pw[g] = __builtin_amdgcn_exp2f(sc[g] - mx);
    psum += pw[g];
  }
  const float denom = wave_sum(psum) + p1;

  // ---- output: channel = lane, this wavefront's keys ----
  float acc = wave == 0 ? p1 * vn : 0.f;
#pragma unroll
  for (int u = 0; u < kPerWave; ++u) {
    const int j = 4 * u + wave;
    const float p = __shfl(pw[u >> 4], j & 63, 64);  // key j sits in group j / 64 = u / 16
    acc = __builtin_fmaf(j < ncached ? p : 0.f, vv[u], acc);
  }
  s_part[wave][lane] = acc;
  __syncthreads();
  if (wave == 0) {
    const float tot = s_part[0][lane] + s_part[1][lane] + s_part[2][lane] + s_part[3][lane];
    o[b * o_sb + h * o_sh + lane] = (__bf16)(tot / denom);
  }
}

// ------------------------------------------------------------------------------------------
// Any head dimension (a multiple of 8, up to 128), fp32 arithmetic: one wavefront per query.
// Not a performance path: it serves the head sizes the MFMA kernels are not built for (the
// reference's own test models have 16-dim heads) and is simple enough to be read as a second
// statement of the same attention.  Lanes run over the keys of the window for the scores and
// over the channels for the output.
// ------------------------------------------------------------------------------------------
constexpr int kAnyMaxDim = 128;
constexpr int kAnyMaxKeys = 192;   // keys a query can see, rounded up to whole wavefront passes (129 -> 3 x 64)

__global__ __launch_bounds__(256) void swa_prefill_anydim_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ k, const __bf16* __restrict__ v,
    __bf16* __restrict__ o, int H, int L, int D, long n_rows, long q_sb, long q_sl, long q_sh, long k_sb, long k_sl,
    long k_sh, long v_sb, long v_sl, long v_sh, long o_sb, long o_sl, long o_sh, int w_left, float scale_log2e,
    __bf16* __restrict__ kc_out, __bf16* __restrict__ vc_out, long c_sb, long c_st, long c_sh) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);  // (b, h, n) flattened, n fastest
  if (row >= n_rows) return;
  const int n = (int)(row % L);
  const int h = (int)((row / L) % H);
  const long b = row / ((long)L * H);
  const __bf16* qr = q + b * q_sb + (long)n * q_sl + h * q_sh;
  const __bf16* kb = k + b * k_sb + h * k_sh;
  const __bf16* vb = v + b * v_sb + h * v_sh;
  const int lo = n - w_left > 0 ? n - w_left : 0;
  const int nkeys = n - lo + 1;  // 1 .. w_left + 1
  // scores: lane j of pass p takes key lo + 64 p + j
  float sc[kAnyMaxKeys / 64];
  float mx = -INFINITY;
#pragma unroll
  for (int p = 0; p < kAnyMaxKeys / 64; ++p) {
    const int j = 64 * p + lane;
    float dot = -INFINITY;
    if (j < nkeys) {
      const __bf16* kr = kb + (long)(lo + j) * k_sl;
      dot = 0.f;
      for (int c = 0; c < D; c += 8) {
        const bf16x8 kk = *reinterpret_cast<const bf16x8*>(kr + c);
        const bf16x8 qq = *reinterpret_cast<const bf16x8*>(qr + c);
#pragma unroll
        for (int i = 0; i < 8; ++i) dot = __builtin_fmaf(to_f32(kk[i]), to_f32(qq[i]), dot);
      }
      dot *= scale_log2e;
    }
    sc[p] = dot;
    mx = fmaxf(mx, dot);
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, 64));
  float psum = 0.f;
#pragma unroll
  for (int p = 0; p < kAnyMaxKeys / 64; ++p) {
    sc[p] = __builtin_amdgcn_exp2f(sc[p] - mx);  // exp2(-inf) = 0 for the lanes without a key
    psum += sc[p];
  }
  const float denom = wave_sum(psum);
  // output: lane c (and c + 64) accumulates its channel over the keys
  float acc[kAnyMaxDim / 64] = {0.f, 0.f};
#pragma unroll
  for (int p = 0; p < kAnyMaxKeys / 64; ++p) {
    const int cnt = nkeys - 64 * p < 64 ? nkeys - 64 * p : 64;
    for (int j = 0; j < cnt; ++j) {
      const float w = __shfl(sc[p], j, 64);
      const __bf16* vr = vb + (long)(lo + 64 * p + j) * v_sl;
#pragma unroll
      for (int u = 0; u < kAnyMaxDim / 64; ++u)
        if (lane + 64 * u < D) acc[u] = __builtin_fmaf(w, to_f32(vr[lane + 64 * u]), acc[u]);
    }
  }
  __bf16* orow = o + b * o_sb + (long)n * o_sl + h * o_sh;
#pragma unroll
  for (int u = 0; u < kAnyMaxDim / 64; ++u)
    if (lane + 64 * u < D) orow[lane + 64 * u] = (__bf16)(acc[u] / denom);
  if (kc_out != nullptr) {  // this token's k and v rows join the cache
    __bf16* kc = kc_out + b * c_sb + (long)n * c_st + h * c_sh;
    __bf16* vc = vc_out + b * c_sb + (long)n * c_st + h * c_sh;
#pragma unroll
    for (int u = 0; u < kAnyMaxDim / 64; ++u)
      if (lane + 64 * u < D) {
        kc[lane + 64 * u] = kb[(long)n * k_sl + lane + 64 * u];
        vc[lane + 64 * u] = vb[(long)n * v_sl + lane + 64 * u];
      }
  }
}

// Decode step for any head dimension: one wavefront per (b, h); cache rows lo .. pos - 1 plus the new
// token, whose k and v are used from registers and written to cache row pos.
__global__ __launch_bounds__(64) void swa_step_anydim_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ k_new, const __bf16* __restrict__ v_new,
    __bf16* __restrict__ kcache, __bf16* __restrict__ vcache, __bf16* __restrict__ o,
    const int32_t* __restrict__ cache_seqlens, int pos_host, int H, int D, int max_seqlen, long q_sb, long q_sh,
    long kn_sb, long kn_sh, long vn_sb, long vn_sh, long o_sb, long o_sh, long c_sb, long c_st, long c_sh, int w_left,
    float scale_log2e) {
  const int lane = threadIdx.x;
  const int b = blockIdx.x / H, h = blockIdx.x % H;
  int pos = cache_seqlens ? cache_seqlens[b] : pos_host;
  pos = __builtin_amdgcn_readfirstlane(pos);
  __bf16* orow = o + b * o_sb + h * o_sh;
  if (pos < 0 || pos >= max_seqlen) {  // see swa_step_kernel: NaN marks what the host cannot be told
#pragma unroll
    for (int u = 0; u < kAnyMaxDim / 64; ++u)
      if (lane + 64 * u < D) orow[lane + 64 * u] = (__bf16)__builtin_nanf("");
    return;
  }
  const __bf16* qr = q + b * q_sb + h * q_sh;
  const __bf16* knr = k_new + b * kn_sb + h * kn_sh;
  const __bf16* vnr = v_new + b * vn_sb + h * vn_sh;
  __bf16* kc = kcache + b * c_sb + h * c_sh;
  __bf16* vc = vcache + b * c_sb + h * c_sh;
  const int lo = pos - w_left > 0 ? pos - w_left : 0;
  const int ncached = pos - lo;  // 0 .. 128
  float sc[2];
  float mx = -INFINITY;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int j = 64 * p + lane;
    float dot = -INFINITY;
    if (j < ncached) {
      const __bf16* kr = kc + (long)(lo + j) * c_st;
      dot = 0.f;
      for (int c = 0; c < D; c += 8) {
        const bf16x8 kk = *reinterpret_cast<const bf16x8*>(kr + c);
        const bf16x8 qq = *reinterpret_cast<const bf16x8*>(qr + c);
#pragma unroll
        for (int i = 0; i < 8; ++i) dot = __builtin_fmaf(to_f32(kk[i]), to_f32(qq[i]), dot);
      }
      dot *= scale_log2e;
    }
    sc[p] = dot;
    mx = fmaxf(mx, dot);
  }
  // the new token: lanes over channels
  float part = 0.f, vn[kAnyMaxDim / 64];
  __bf16 kn[kAnyMaxDim / 64];
#pragma unroll
  for (int u = 0; u < kAnyMaxDim / 64; ++u) {
    vn[u] = 0.f;
    kn[u] = (__bf16)0.f;
    if (lane + 64 * u < D) {
      kn[u] = knr[lane + 64 * u];
      vn[u] = to_f32(vnr[lane + 64 * u]);
      part = __builtin_fmaf(to_f32(qr[lane + 64 * u]), to_f32(kn[u]), part);
    }
  }
  const float self = wave_sum(part) * scale_log2e;
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, 64));
  mx = fmaxf(mx, self);
  float psum = 0.f;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    sc[p] = __builtin_amdgcn_exp2f(sc[p] - mx);
    psum += sc[p];
  }
  const float pself = __builtin_amdgcn_exp2f(self - mx);
  const float denom = wave_sum(psum) + pself;
  float acc[kAnyMaxDim / 64];
#pragma unroll
  for (int u = 0; u < kAnyMaxDim / 64; ++u) acc[u] = pself * vn[u];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int cnt = ncached - 64 * p < 64 ? ncached - 64 * p : 64;
    for (int j = 0; j < cnt; ++j) {
      const float w = __shfl(sc[p], j, 64);
      const __bf16* vr = vc + (long)(lo + 64 * p + j) * c_st;
#pragma unroll
      for (int u = 0; u < kAnyMaxDim / 64; ++u)
        if (lane + 64 * u < D) acc[u] = __builtin_fmaf(w, to_f32(vr[lane + 64 * u]), acc[u]);
    }
  }
#pragma unroll
  for (int u = 0; u < kAnyMaxDim / 64; ++u)
    if (lane + 64 * u < D) {
      orow[lane + 64 * u] = (__bf16)(acc[u] / denom);
      kc[(long)pos * c_st + lane + 64 * u] = kn[u];
      vc[(long)pos * c_st + lane + 64 * u] = (__bf16)vn[u];
    }
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

constexpr int kMaxDevices = 64;
// kernels asking for more than 64 KB of LDS have to be told once per device that they may
static std::atomic<bool> g_big_lds_allowed[kMaxDevices][2 /*ROPE*/][2 /*NB - 2*/][3 /*G = 1, 2, 4*/];

}  // namespace based

extern "C" BASED_API int based_swa_prefill(const void* q, const void* k, const void* v, void* o,
                                           int64_t B, int64_t H, int64_t L,
                                           int64_t q_sb, int64_t q_sl, int64_t q_sh,
                                           int64_t k_sb, int64_t k_sl, int64_t k_sh,
                                           int64_t v_sb, int64_t v_sl, int64_t v_sh,
                                           int64_t o_sb, int64_t o_sl, int64_t o_sh,
                                           int w_left, float scale,
                                           const float* rope_cos, const float* rope_sin, int64_t rope_len,
                                           void* kcache_out, void* vcache_out,
                                           int64_t c_sb, int64_t c_st, int64_t c_sh, int64_t max_seqlen,
                                           int io_dtype, void* stream) {
  using namespace based;
  BASED_REQUIRE(q && k && v && o, BASED_ERR_ARG, "swa_prefill: null pointer argument");
  BASED_REQUIRE((rope_cos == nullptr) == (rope_sin == nullptr), BASED_ERR_ARG,
                "swa_prefill: rotary tables must be given together");
  if (rope_cos)
    BASED_REQUIRE(rope_len >= L, BASED_ERR_ARG, "swa_prefill: rotary tables hold %ld positions, need %ld",
                  (long)rope_len, (long)L);
  BASED_REQUIRE((kcache_out == nullptr) == (vcache_out == nullptr), BASED_ERR_ARG,
                "swa_prefill: cache outputs must be given together");
  if (kcache_out) {
    BASED_REQUIRE(L <= max_seqlen, BASED_ERR_SHAPE, "swa_prefill: %ld tokens do not fit a cache of %ld rows",
                  (long)L, (long)max_seqlen);
    BASED_REQUIRE(c_sb % 8 == 0 && c_st % 8 == 0 && c_sh % 8 == 0, BASED_ERR_ALIGN,
                  "swa_prefill: cache strides must be multiples of 8 elements");
    BASED_REQUIRE(aligned16(kcache_out) && aligned16(vcache_out), BASED_ERR_ALIGN,
                  "swa_prefill: caches must be 16-byte aligned");
  }
  BASED_REQUIRE(B >= 0 && H > 0 && L >= 0, BASED_ERR_ARG, "swa_prefill: bad sizes");
  BASED_REQUIRE(io_dtype == BASED_BF16, BASED_ERR_DTYPE, "swa_prefill: only bf16 is supported");
  BASED_REQUIRE(w_left >= 0 && w_left <= 128, BASED_ERR_SHAPE,
                "swa_prefill: left window %d unsupported (0..128)", w_left);
  BASED_REQUIRE(H < 65536 && B < 65536 && L < (1ll << 31) - 64, BASED_ERR_SHAPE,
                "swa_prefill: grid too large");
  const int64_t strides[] = {q_sb, q_sl, q_sh, k_sb, k_sl, k_sh, v_sb, v_sl, v_sh, o_sb, o_sl, o_sh};
  for (int64_t s : strides)
    BASED_REQUIRE(s % 8 == 0, BASED_ERR_ALIGN, "swa_prefill: strides must be multiples of 8 elements");
  BASED_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(o), BASED_ERR_ALIGN,
                "swa_prefill: tensors must be 16-byte aligned");
  if (B == 0 || L == 0) return BASED_OK;
  const int64_t n_tiles = (L + kQTile - 1) / kQTile;
  BASED_REQUIRE(B * H * n_tiles < (1ll << 31), BASED_ERR_SHAPE, "swa_prefill: grid too large");
  // Heads that are neighbours in every tensor (the packed qkv layout) share a workgroup, so that
  // every load and store instruction covers pieces of 128 G bytes.  Two-block ring: four heads
  // (16 wavefronts, 160 KB of LDS: one workgroup per compute unit; 57.1 -> 53.9 us at B=8, H=16,
  // L=4096 against two heads in each of two workgroups), else two.  Three-block ring: two heads
  // (112 KB, one workgroup of 8 wavefronts per unit, whose registers allow the loop unrolled over
  // the ring's positions: see the kernel), one head (three workgroups of 4 wavefronts) only where
  // the heads are not neighbours.
  const bool rope = rope_cos != nullptr;
  const int nb = w_left > 64 ? 3 : 2;
  const bool pair = H % 2 == 0 && q_sh == 64 && k_sh == 64 && v_sh == 64 && o_sh == 64 &&
                    (!kcache_out || c_sh == 64);
  const int g = !pair ? 1 : (nb == 2 && H % 4 == 0 ? 4 : 2);
  // Consecutive query tiles of one (batch, head) are walked by one workgroup (the keys to the left
  // of a tile are the previous tile's own keys, already staged).  Runs are as long as still gives
  // every resident slot of the GPU one run: 256 compute units x the wavefront quartets that fit
  // one (4 by registers; for the three-block ring, by LDS, 3 of one head or 2 of a pair; 3 for the
  // single-head rotary variant).
  const int64_t slots = 256 * (nb == 3 ? (g == 2 ? 2 : 3) : ((g == 1 && rope) ? 3 : 4));
  int64_t want_runs = slots / (B * H);
  want_runs = want_runs < 1 ? 1 : (want_runs > n_tiles ? n_tiles : want_runs);
  const int64_t run_tiles = (n_tiles + want_runs - 1) / want_runs;
  const int64_t runs_per_seq = (n_tiles + run_tiles - 1) / run_tiles;
  dim3 grid((unsigned)(B * (H / g) * runs_per_seq)), block(256 * g);
  using Kern = void (*)(const __bf16*, const __bf16*, const __bf16*, __bf16*, int, int, int, int, long, long, long, long,
                        long, long, long, long, long, long, long, long, int, float, const float*, const float*, __bf16*,
                        __bf16*, long, long, long);
  Kern kern;
  if (nb == 3 && g == 2) kern = rope ? swa_prefill_kernel<true, 3, 2> : swa_prefill_kernel<false, 3, 2>;
  else if (nb == 3) kern = rope ? swa_prefill_kernel<true, 3, 1> : swa_prefill_kernel<false, 3, 1>;
  else if (g == 4) kern = rope ? swa_prefill_kernel<true, 2, 4> : swa_prefill_kernel<false, 2, 4>;
  else if (g == 2) kern = rope ? swa_prefill_kernel<true, 2, 2> : swa_prefill_kernel<false, 2, 2>;
  else kern = rope ? swa_prefill_kernel<true, 2, 1> : swa_prefill_kernel<false, 2, 1>;
  const size_t lds = (size_t)g * swa_head_lds_bytes(nb, g);
  if (lds > 64 * 1024) {
    int dev = 0;
    BASED_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices, BASED_ERR_LAUNCH,
                  "swa_prefill: cannot identify the current device");
    std::atomic<bool>& allowed = g_big_lds_allowed[dev][rope][nb - 2][g == 4 ? 2 : g - 1];
    if (!allowed.load(std::memory_order_acquire)) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      BASED_REQUIRE(e == hipSuccess, BASED_ERR_LAUNCH, "swa_prefill: cannot raise the LDS limit to %zu bytes: %s", lds,
                    hipGetErrorString(e));
      allowed.store(true, std::memory_order_release);
    }
  }
  hipLaunchKernelGGL(kern, grid, block, lds, static_cast<hipStream_t>(stream),
                     (const __bf16*)q, (const __bf16*)k, (const __bf16*)v, (__bf16*)o, (int)H, (int)L,
                     (int)n_tiles, (int)run_tiles, q_sb, q_sl, q_sh, k_sb, k_sl, k_sh, v_sb, v_sl, v_sh, o_sb,
                     o_sl, o_sh, w_left, scale * 1.4426950408889634f, rope_cos, rope_sin,
                     (__bf16*)kcache_out, (__bf16*)vcache_out, c_sb, c_st, c_sh);
  return check_launch("swa_prefill");
}

extern "C" BASED_API int based_swa_step(const void* q, const void* k_new, const void* v_new,
                                        void* kcache, void* vcache, void* o,
                                        const int32_t* cache_seqlens, int64_t pos_host,
                                        int64_t B, int64_t H, int64_t max_seqlen,
                                        int64_t q_sb, int64_t q_sh, int64_t kn_sb, int64_t kn_sh,
                                        int64_t vn_sb, int64_t vn_sh, int64_t o_sb, int64_t o_sh,
                                        int64_t c_sb, int64_t c_st, int64_t c_sh,
                                        int w_left, float scale,
                                        const float* rope_cos, const float* rope_sin, int64_t rope_len,
                                        int io_dtype, void* stream) {
  using namespace based;
  BASED_REQUIRE(q && k_new && v_new && kcache && vcache && o, BASED_ERR_ARG,
                "swa_step: null pointer argument");
  BASED_REQUIRE((rope_cos == nullptr) == (rope_sin == nullptr), BASED_ERR_ARG,
                "swa_step: rotary tables must be given together");
  if (rope_cos) {
    BASED_REQUIRE(rope_len > 0 && rope_len < (1ll << 31), BASED_ERR_ARG, "swa_step: bad rotary table length");
    if (!cache_seqlens)
      BASED_REQUIRE(pos_host < rope_len, BASED_ERR_ARG, "swa_step: position %ld beyond the rotary table (%ld rows)",
                    (long)pos_host, (long)rope_len);
  }
  BASED_REQUIRE(B >= 0 && H > 0 && max_seqlen > 0, BASED_ERR_ARG, "swa_step: bad sizes");
  BASED_REQUIRE(io_dtype == BASED_BF16, BASED_ERR_DTYPE, "swa_step: only bf16 is supported");
  BASED_REQUIRE(w_left >= 0 && w_left <= 128, BASED_ERR_SHAPE,
                "swa_step: left window %d unsupported (0..128)", w_left);
  BASED_REQUIRE(max_seqlen < (1ll << 31) && B * H < (1ll << 31), BASED_ERR_SHAPE, "swa_step: sizes too large");
  if (!cache_seqlens)
    BASED_REQUIRE(pos_host >= 0 && pos_host < max_seqlen, BASED_ERR_ARG,
                  "swa_step: position %ld outside the cache (max_seqlen %ld)", (long)pos_host,
                  (long)max_seqlen);
  BASED_REQUIRE(c_sb % 8 == 0 && c_st % 8 == 0 && c_sh % 8 == 0 && q_sb % 8 == 0 && q_sh % 8 == 0,
                BASED_ERR_ALIGN, "swa_step: cache and q strides must be multiples of 8 elements");
  BASED_REQUIRE(aligned16(kcache) && aligned16(q), BASED_ERR_ALIGN,
                "swa_step: kcache and q must be 16-byte aligned");
  if (B == 0) return BASED_OK;
  hipLaunchKernelGGL(w_left > 64 ? swa_step_kernel<2> : swa_step_kernel<1>, dim3((unsigned)(B * H)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), (const __bf16*)q, (const __bf16*)k_new,
                     (const __bf16*)v_new, (__bf16*)kcache, (__bf16*)vcache, (__bf16*)o, cache_seqlens,
                     (int)pos_host, (int)H, (int)max_seqlen, q_sb, q_sh, kn_sb, kn_sh, vn_sb, vn_sh,
                     o_sb, o_sh, c_sb, c_st, c_sh, w_left, scale * 1.4426950408889634f, rope_cos, rope_sin,
                     (int)rope_len);
  return check_launch("swa_step");
}

extern "C" BASED_API int based_swa_prefill_anydim(const void* q, const void* k, const void* v, void* o,
                                                  int64_t B, int64_t H, int64_t L, int64_t D,
                                                  int64_t q_sb, int64_t q_sl, int64_t q_sh,
                                                  int64_t k_sb, int64_t k_sl, int64_t k_sh,
                                                  int64_t v_sb, int64_t v_sl, int64_t v_sh,
                                                  int64_t o_sb, int64_t o_sl, int64_t o_sh,
                                                  int w_left, float scale,
                                                  void* kcache_out, void* vcache_out,
                                                  int64_t c_sb, int64_t c_st, int64_t c_sh, int64_t max_seqlen,
                                                  int io_dtype, void* stream) {
  using namespace based;
  BASED_REQUIRE(q && k && v && o, BASED_ERR_ARG, "swa_prefill_anydim: null pointer argument");
  BASED_REQUIRE((kcache_out == nullptr) == (vcache_out == nullptr), BASED_ERR_ARG,
                "swa_prefill_anydim: cache outputs must be given together");
  if (kcache_out)
    BASED_REQUIRE(L <= max_seqlen, BASED_ERR_SHAPE, "swa_prefill_anydim: %ld tokens do not fit a cache of %ld rows",
                  (long)L, (long)max_seqlen);
  BASED_REQUIRE(B >= 0 && H > 0 && L >= 0, BASED_ERR_ARG, "swa_prefill_anydim: bad sizes");
  BASED_REQUIRE(io_dtype == BASED_BF16, BASED_ERR_DTYPE, "swa_prefill_anydim: only bf16 is supported");
  BASED_REQUIRE(D >= 8 && D <= kAnyMaxDim && D % 8 == 0, BASED_ERR_SHAPE,
                "swa_prefill_anydim: head dim %ld unsupported (multiples of 8 up to %d)", (long)D, kAnyMaxDim);
  BASED_REQUIRE(w_left >= 0 && w_left <= 128, BASED_ERR_SHAPE, "swa_prefill_anydim: left window %d unsupported (0..128)",
                w_left);
  const int64_t strides[] = {q_sb, q_sl, q_sh, k_sb, k_sl, k_sh, v_sb, v_sl, v_sh};
  for (int64_t st : strides)
    BASED_REQUIRE(st % 8 == 0, BASED_ERR_ALIGN, "swa_prefill_anydim: q, k, v strides must be multiples of 8 elements");
  BASED_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v), BASED_ERR_ALIGN,
                "swa_prefill_anydim: q, k, v must be 16-byte aligned");
  if (B == 0 || L == 0) return BASED_OK;
  const int64_t n_rows = B * H * L;
  BASED_REQUIRE((n_rows + 3) / 4 < (1ll << 31) && L < (1ll << 31), BASED_ERR_SHAPE, "swa_prefill_anydim: grid too large");
  hipLaunchKernelGGL(swa_prefill_anydim_kernel, dim3((unsigned)((n_rows + 3) / 4)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), (const __bf16*)q, (const __bf16*)k, (const __bf16*)v, (__bf16*)o,
                     (int)H, (int)L, (int)D, (long)n_rows, q_sb, q_sl, q_sh, k_sb, k_sl, k_sh, v_sb, v_sl, v_sh, o_sb, o_sl,
                     o_sh, w_left, scale * 1.4426950408889634f, (__bf16*)kcache_out, (__bf16*)vcache_out, c_sb, c_st,
                     c_sh);
  return check_launch("swa_prefill_anydim");
}

extern "C" BASED_API int based_swa_step_anydim(const void* q, const void* k_new, const void* v_new,
                                               void* kcache, void* vcache, void* o,
                                               const int32_t* cache_seqlens, int64_t pos_host,
                                               int64_t B, int64_t H, int64_t D, int64_t max_seqlen,
                                               int64_t q_sb, int64_t q_sh, int64_t kn_sb, int64_t kn_sh,
                                               int64_t vn_sb, int64_t vn_sh, int64_t o_sb, int64_t o_sh,
                                               int64_t c_sb, int64_t c_st, int64_t c_sh,
                                               int w_left, float scale, int io_dtype, void* stream) {
  using namespace based;
  BASED_REQUIRE(q && k_new && v_new && kcache && vcache && o, BASED_ERR_ARG, "swa_step_anydim: null pointer argument");
  BASED_REQUIRE(B >= 0 && H > 0 && max_seqlen > 0, BASED_ERR_ARG, "swa_step_anydim: bad sizes");
  BASED_REQUIRE(io_dtype == BASED_BF16, BASED_ERR_DTYPE, "swa_step_anydim: only bf16 is supported");
  BASED_REQUIRE(D >= 8 && D <= kAnyMaxDim && D % 8 == 0, BASED_ERR_SHAPE,
                "swa_step_anydim: head dim %ld unsupported (multiples of 8 up to %d)", (long)D, kAnyMaxDim);
  BASED_REQUIRE(w_left >= 0 && w_left <= 128, BASED_ERR_SHAPE, "swa_step_anydim: left window %d unsupported (0..128)",
                w_left);
  BASED_REQUIRE(max_seqlen < (1ll << 31) && B * H < (1ll << 31), BASED_ERR_SHAPE, "swa_step_anydim: sizes too large");
  if (!cache_seqlens)
    BASED_REQUIRE(pos_host >= 0 && pos_host < max_seqlen, BASED_ERR_ARG,
                  "swa_step_anydim: position %ld outside the cache (max_seqlen %ld)", (long)pos_host, (long)max_seqlen);
  BASED_REQUIRE(c_sb % 8 == 0 && c_st % 8 == 0 && c_sh % 8 == 0 && q_sb % 8 == 0 && q_sh % 8 == 0, BASED_ERR_ALIGN,
                "swa_step_anydim: cache and q strides must be multiples of 8 elements");
  BASED_REQUIRE(aligned16(kcache) && aligned16(q), BASED_ERR_ALIGN, "swa_step_anydim: kcache and q must be 16-byte aligned");
  if (B == 0) return BASED_OK;
  hipLaunchKernelGGL(swa_step_anydim_kernel, dim3((unsigned)(B * H)), dim3(64), 0, static_cast<hipStream_t>(stream),
                     (const __bf16*)q, (const __bf16*)k_new, (const __bf16*)v_new, (__bf16*)kcache, (__bf16*)vcache,
                     (__bf16*)o, cache_seqlens, (int)pos_host, (int)H, (int)D, (int)max_seqlen, q_sb, q_sh, kn_sb, kn_sh,
                     vn_sb, vn_sh, o_sb, o_sh, c_sb, c_st, c_sh, w_left, scale * 1.4426950408889634f);
  return check_launch("swa_step_anydim");
}
