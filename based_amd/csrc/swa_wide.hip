// Sliding-window causal softmax attention for head dims other than 64 (any multiple of 8 up to
// 128: 112 and 128 are the released 1B / 1.3B shapes) and for every rotary layout the reference's
// constructor admits (rotary over a leading part of the head, half-split or interleaved pairs).
// Same algorithm as the 64-channel kernels of swa.hip, with LDS rows of 256 bytes (128 channels,
// zero padded past the head dim):
//
// Prefill.  Four wavefronts cover 64 consecutive queries of one (batch, head); wavefront w owns
// queries [q0 + 16 w, q0 + 16 w + 16) and sees the staged keys 16 w .. 16 w + 16 NT - 1 of a ring
// of blocks of 64 K rows and 64 V rows (NB = 2: up to 64 keys to the left, NB = 3: up to 128).
// With NB = 3 a workgroup is eight wavefronts on two neighbouring tiles that share the blocks to
// their left (a ring of four blocks).
//   S^T = K Q^T   : NT key tiles x 2 or 4 MFMA 16x16x32 (head dims up to 64 / 128); K and Q rows are staged in LDS
//                   (rotated on the way in), a lane's operand = 8 consecutive bf16 of one row.
//   softmax       : whole window in one pass, lane <-> query, registers <-> keys.
//   O^T = V^T P^T : P from the accumulator registers, V^T by the transposing LDS read; the
//                   16 x D output tile is staged in the wavefront's own 16 query rows so that
//                   every lane stores 16 bytes of a full row.
// Rows travel global -> registers -> LDS one tile ahead, every load unconditional (rows outside
// the sequence are fetched from its nearest row and masked; pieces past the head dim from piece 0
// and zeroed).  A thread moves, per row, the TWO 16-byte pieces that the rotation pairs up.
//
// Decode.  One workgroup of four wavefronts per (batch, head) against the last w_left + 1 rows of
// the linear cache, every load issued up front.
#include "common.hpp"

#include <atomic>

namespace based {

constexpr int kWQTile = 64;          // queries per workgroup and tile; rows per ring block
constexpr int kWRowBytes = 256;      // LDS row: 128 channels
constexpr int kWMaxDim = 128;
constexpr int kRopeNone = 0, kRopeHalf = 1, kRopeInterleaved = 2;

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// Piece p (16 bytes, 0..15) of LDS row r sits at:
//   K and Q rows (MFMA operands: 16 consecutive rows x the same piece): p ^ (r & 15), sixteen
//   different pieces = all 64 banks;
//   V rows (transposing read: 8 consecutive rows x two neighbouring pieces per half-wavefront):
//   the piece PAIR index is swizzled, ((p >> 1) ^ (r & 7)) << 1 | (p & 1).
__device__ __forceinline__ int wide_swz_k(int row, int p) { return p ^ (row & 15); }
__device__ __forceinline__ int wide_swz_v(int row, int p) { return ((((p >> 1) ^ (row & 7)) << 1) | (p & 1)); }

// half-split pairs: element j of `lo` (channel c) with element j of `hi` (channel c + R/2)
__device__ __forceinline__ void wide_rotate_half(u32x4& lo, u32x4& hi, const f32x4 (&cs)[2], const f32x4 (&sn)[2]) {
  u32x4 out_lo, out_hi;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    float o1[2], o2[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int j = 2 * d + e;
      const float x1 = bf16_bits_to_f32(e == 0 ? (lo[d] & 0xFFFFu) : (lo[d] >> 16));
      const float x2 = bf16_bits_to_f32(e == 0 ? (hi[d] & 0xFFFFu) : (hi[d] >> 16));
      const float c = cs[j >> 2][j & 3], s = sn[j >> 2][j & 3];
      o1[e] = x1 * c - x2 * s;
      o2[e] = x1 * s + x2 * c;
    }
    out_lo[d] = pack_bf16(o1[0], o1[1]);
    out_hi[d] = pack_bf16(o2[0], o2[1]);
  }
  lo = out_lo;
  hi = out_hi;
}
// interleaved pairs: the two halves of dword d of a piece, frequency d of the piece's four
__device__ __forceinline__ void wide_rotate_interleaved(u32x4& x, const f32x4& cs, const f32x4& sn) {
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const float x1 = bf16_bits_to_f32(x[d] & 0xFFFFu), x2 = bf16_bits_to_f32(x[d] >> 16);
    x[d] = pack_bf16(x1 * cs[d] - x2 * sn[d], x1 * sn[d] + x2 * cs[d]);
  }
}

// two rows' worth of pieces per thread on their way from global memory to LDS
struct WideRows {
  u32x4 kp[2][2], vp[2][2], qp[2][2];  // [row][piece a / b]
  f32x4 cs[2][2], sn[2][2];            // rotary factors of the row's position (RMODE != 0)
};

// ring of nb - 1 + qt blocks of K rows and of V rows, qt blocks of query rows
constexpr int wide_lds_bytes(int nb, int qt) { return (2 * (nb - 1 + qt) + qt) * kWQTile * kWRowBytes; }

// RMODE: rotary layout (kRopeNone / kRopeHalf / kRopeInterleaved) over the first R channels, cos/sin
// tables of R/2 frequencies per position (slide_attention.py:346-355,553-556); kc_out / vc_out
// (optional): the (rotated) K rows and the V rows of this call also go to a KV cache
// (_update_kv_cache, slide_attention.py:255-281).
// NDS: contraction steps of 32 channels (head dims up to 32 NDS); a compile-time count keeps the
// products free of branches, so that the operand reads of one MFMA travel under the others.
// QT: tiles of 64 queries a workgroup of 4 QT wavefronts works on at a time (run_tiles is a
// multiple of it).  With the three-block window a lone tile's ring fills a compute unit's LDS
// share with four wavefronts; two tiles side by side share the window's blocks (four ring blocks
// instead of twice three: 160 KB), so that every SIMD has two wavefronts to switch between.
template <int RMODE, int NB, int NDS, int QT>
__global__ __launch_bounds__(256 * QT, QT == 2 || NB == 2 ? 2 : 1) void swa_prefill_wide_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ k, const __bf16* __restrict__ v,
    __bf16* __restrict__ o, int H, int L, int D, int n_tiles, int run_tiles, long q_sb, long q_sl, long q_sh,
    long k_sb, long k_sl, long k_sh, long v_sb, long v_sl, long v_sh, long o_sb, long o_sl, long o_sh,
    int w_left, float scale_log2e, const float* __restrict__ rope_cos, const float* __restrict__ rope_sin, int R,
    __bf16* __restrict__ kc_out, __bf16* __restrict__ vc_out, long c_sb, long c_st, long c_sh) {
  constexpr int NT = 4 * (NB - 1) + 1;   // key tiles of 16 a wavefront sees
  constexpr int NS = (NT + 1) / 2;       // key slabs of 32 in the second product (last one half empty)
  static_assert((NB - 1) % QT == 0, "the keys to the left are loaded in pieces of QT blocks");
  constexpr int NBR = NB - 1 + QT;       // ring blocks
  constexpr int kSuper = QT * kWQTile;   // queries (and new key rows) per step of the workgroup
  constexpr int kOffV = NBR * kWQTile * kWRowBytes;
  constexpr int kOffQ = 2 * kOffV;
  extern __shared__ __align__(16) unsigned char swa_wide_lds[];
  unsigned char* const lds = swa_wide_lds;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w8 = __builtin_amdgcn_readfirstlane(tid >> 6);  // which 16 of the step's 64 QT queries
  const int wt = w8 >> 2;                                   // which tile of the step
  const int wq = w8 & 3;                                    // which 16 of the tile's 64 queries
  const int col = lane & 15;
  const int grp = lane >> 4;
  const int np = D >> 3;            // live 16-byte pieces of a row
  constexpr int NET = 2 * NDS;      // output channel tiles of 16 (a tile past the head dim works on zeros)
  const bool whole_lines = (D & 63) == 0 && (o_sh & 63) == 0 && (o_sl & 63) == 0;

  // Work item: a run of consecutive query tiles of one (batch, head).  The heads of one run of
  // tokens are consecutive items and consecutive items are laid along one XCD (workgroup ids are
  // dealt to the 8 XCDs round-robin): a token's rows of all heads are one contiguous piece of
  // memory, and head rows of 224 bytes (head dim 112) start and end inside 128-byte lines that
  // two neighbouring heads share; the neighbours then read and write those lines behind the same
  // L2 at about the same time (measured with a streaming probe: 128-byte accesses into 224-byte
  // head rows from unrelated workgroups run at 2.4 TB/s, half the rate of aligned rows).
  const int runs_per_seq = (n_tiles + run_tiles - 1) / run_tiles;
  const unsigned n_item = gridDim.x;
  const unsigned item = n_item % 8 == 0 ? (blockIdx.x % 8) * (n_item / 8) + blockIdx.x / 8 : blockIdx.x;
  const int h = (int)(item % (unsigned)H);
  const unsigned rest = item / (unsigned)H;
  const int run = (int)(rest % (unsigned)runs_per_seq), b = (int)(rest / (unsigned)runs_per_seq);
  const int tile_begin = run * run_tiles;
  const int tile_end = tile_begin + run_tiles < n_tiles ? tile_begin + run_tiles : n_tiles;

  // Pieces moved by this thread: rows 16 w8 + lane / 8 (+ 8) of a step's 64 QT, piece pair `slot` = lane % 8.
  //   half-split rotary: slot s < R/16 is the pair (s, s + R/16) that the rotation combines
  //     (channels c and c + R/2); the other slots carry the unrotated pieces past R, two by two;
  //   otherwise: slot s = pieces 2 s, 2 s + 1 (interleaved pairs sit inside one piece).
  // Frequencies of slot s in either layout: 8 s .. 8 s + 7.
  const int slot = lane & 7;
  const int r16 = R >> 4;
  int pa, pb;
  if constexpr (RMODE == kRopeHalf) {
    if (slot < r16) {
      pa = slot;
      pb = slot + r16;
    } else {
      pa = (R >> 3) + 2 * (slot - r16);
      pb = pa + 1;
    }
  } else {
    pa = 2 * slot;
    pb = pa + 1;
  }
  const bool rot = RMODE != kRopeNone && slot < r16;
  const bool va = pa < np, vb = pb < np;
  const int pa_ld = va ? 8 * pa : 0, pb_ld = vb ? 8 * pb : 0;   // element offsets of the loads (always inside the row)
  const int row_lo = 16 * w8 + (lane >> 3);
  const __bf16* const q_mv = q + b * q_sb + h * q_sh;
  const __bf16* const k_mv = k + b * k_sb + h * k_sh;
  const __bf16* const v_mv = v + b * v_sb + h * v_sh;
  __bf16* kc_mv = nullptr;
  __bf16* vc_mv = nullptr;
  if (kc_out != nullptr) {
    kc_mv = kc_out + b * c_sb + h * c_sh;
    vc_mv = vc_out + b * c_sb + h * c_sh;
  }
  __bf16* const o_my = o + b * o_sb + h * o_sh;
  const int half_r = R >> 1;
  const int f_ld = rot ? 8 * slot : 0;

  auto load_rows = [&](int key0, WideRows& r, bool with_q) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      int key = key0 + row_lo + 8 * i;
      key = key < 0 ? 0 : (key < L ? key : L - 1);
      r.kp[i][0] = *reinterpret_cast<const u32x4*>(k_mv + (long)key * k_sl + pa_ld);
      r.kp[i][1] = *reinterpret_cast<const u32x4*>(k_mv + (long)key * k_sl + pb_ld);
      r.vp[i][0] = *reinterpret_cast<const u32x4*>(v_mv + (long)key * v_sl + pa_ld);
      r.vp[i][1] = *reinterpret_cast<const u32x4*>(v_mv + (long)key * v_sl + pb_ld);
      if (with_q) {  // a literal at every call
        r.qp[i][0] = *reinterpret_cast<const u32x4*>(q_mv + (long)key * q_sl + pa_ld);
        r.qp[i][1] = *reinterpret_cast<const u32x4*>(q_mv + (long)key * q_sl + pb_ld);
      }
      if constexpr (RMODE != kRopeNone) {
        const f32x4* c4 = reinterpret_cast<const f32x4*>(rope_cos + (long)key * half_r + f_ld);
        const f32x4* s4 = reinterpret_cast<const f32x4*>(rope_sin + (long)key * half_r + f_ld);
        r.cs[i][0] = c4[0];
        r.cs[i][1] = c4[1];
        r.sn[i][0] = s4[0];
        r.sn[i][1] = s4[1];
      }
    }
  };
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  // own_rows: the rows are the step's own keys (they also carry its queries and go to the cache);
  // they go to the QT ring blocks from blk on
  auto store_rows = [&](int blk, int key0, WideRows& r, bool own_rows) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if constexpr (RMODE == kRopeHalf) {
        if (rot) {
          wide_rotate_half(r.kp[i][0], r.kp[i][1], r.cs[i], r.sn[i]);
          if (own_rows) wide_rotate_half(r.qp[i][0], r.qp[i][1], r.cs[i], r.sn[i]);
        }
      }
      if constexpr (RMODE == kRopeInterleaved) {
        if (rot) {
          wide_rotate_interleaved(r.kp[i][0], r.cs[i][0], r.sn[i][0]);
          wide_rotate_interleaved(r.kp[i][1], r.cs[i][1], r.sn[i][1]);
          if (own_rows) {
            wide_rotate_interleaved(r.qp[i][0], r.cs[i][0], r.sn[i][0]);
            wide_rotate_interleaved(r.qp[i][1], r.cs[i][1], r.sn[i][1]);
          }
        }
      }
      // pieces past the head dim are zero in LDS (they take part in the products)
      if (!va) r.kp[i][0] = r.vp[i][0] = r.qp[i][0] = zero4;
      if (!vb) r.kp[i][1] = r.vp[i][1] = r.qp[i][1] = zero4;
      const int lrow = row_lo + 8 * i;
      int rblk = blk + (lrow >> 6);
      rblk = rblk >= NBR ? rblk - NBR : rblk;
      const int row = rblk * kWQTile + (lrow & (kWQTile - 1));
      *reinterpret_cast<u32x4*>(lds + row * kWRowBytes + (wide_swz_k(lrow, pa) << 4)) = r.kp[i][0];
      *reinterpret_cast<u32x4*>(lds + row * kWRowBytes + (wide_swz_k(lrow, pb) << 4)) = r.kp[i][1];
      *reinterpret_cast<u32x4*>(lds + kOffV + row * kWRowBytes + (wide_swz_v(lrow, pa) << 4)) = r.vp[i][0];
      *reinterpret_cast<u32x4*>(lds + kOffV + row * kWRowBytes + (wide_swz_v(lrow, pb) << 4)) = r.vp[i][1];
      if (own_rows) {
        *reinterpret_cast<u32x4*>(lds + kOffQ + lrow * kWRowBytes + (wide_swz_k(lrow, pa) << 4)) = r.qp[i][0];
        *reinterpret_cast<u32x4*>(lds + kOffQ + lrow * kWRowBytes + (wide_swz_k(lrow, pb) << 4)) = r.qp[i][1];
      }
      const int key = key0 + lrow;
      if (own_rows && kc_mv != nullptr && key < L) {
        if (va) {
          *reinterpret_cast<u32x4*>(kc_mv + (long)key * c_st + 8 * pa) = r.kp[i][0];
          *reinterpret_cast<u32x4*>(vc_mv + (long)key * c_st + 8 * pa) = r.vp[i][0];
        }
        if (vb) {
          *reinterpret_cast<u32x4*>(kc_mv + (long)key * c_st + 8 * pb) = r.kp[i][1];
          *reinterpret_cast<u32x4*>(vc_mv + (long)key * c_st + 8 * pb) = r.vp[i][1];
        }
      }
    }
  };

  int q0 = tile_begin * kWQTile;
  WideRows pre;
  {
    // first step: own rows in blocks 0 .. QT - 1, the keys 64 QT a to the left in the blocks from
    // NBR - QT a on (one round trip)
    constexpr int kLeft = (NB - 1) / QT;
    WideRows left[kLeft];
#pragma unroll
    for (int a = 1; a <= kLeft; ++a) load_rows(q0 - a * kSuper, left[a - 1], false);
    load_rows(q0, pre, true);
#pragma unroll
    for (int a = 1; a <= kLeft; ++a) store_rows(NBR - a * QT, q0 - a * kSuper, left[a - 1], false);
    store_rows(0, q0, pre, true);
  }
  if (tile_begin + QT < tile_end) load_rows(q0 + kSuper, pre, true);  // travels while this step is computed
  // The three-block ring leaves room for one workgroup per compute unit (112 KB of LDS), i.e. one
  // wavefront per SIMD with the whole register file to itself and nobody to cover its memory
  // round trips: it keeps the rows of TWO tiles in flight (a second register set).
  // (two wavefronts per SIMD have 256 registers each: the rotary factors of a second set do not fit)
  constexpr int DEPTH = NB == 3 && !(QT == 2 && RMODE != kRopeNone) ? 2 : 1;
  WideRows pre2;
  if constexpr (DEPTH == 2)
    if (tile_begin + 2 * QT < tile_end) load_rows(q0 + 2 * kSuper, pre2, true);

  // lane-constant parts of the operand addresses (a tile's rows start at multiples of 16, so
  // row & 15 == col for the operand rows and row & 7 == vt_row & 7 for the transposed ones)
  const int k_lane = col * kWRowBytes;
  const int vt_row = 4 * grp + (col >> 2);
  const int v_lane = vt_row * kWRowBytes + 8 * (col & 1);
  const int v_half = (col & 3) >> 1;

  const int i_win = w_left >= 64 * (NB - 1) + 15 ? 0 : (64 * (NB - 1) + 30 - w_left) >> 4;
  int own = 0;  // ring block with keys [q0, q0 + 64); block own + QT (mod NBR) is the oldest
  // one step of QT tiles; `nxt` holds the rows of the next step and is refilled with those DEPTH steps later
  auto do_tile = [&](int tile, WideRows& nxt) {
    const int oldest = own + QT >= NBR ? own + QT - NBR : own + QT;
    const int x0 = 64 * wt + 16 * wq;   // first staged key this wavefront sees = its first query's place in the step
    const int n0 = q0 + x0;
    const int n = n0 + col;
    auto ring_row = [&](int x) {  // staged key index x (0 .. 64 NBR - 1 <-> key q0 - 64 (NB - 1) + x) -> ring row
      int blk = oldest + (x >> 6);
      blk = blk >= NBR ? blk - NBR : blk;
      return blk * kWQTile + (x & (kWQTile - 1));
    };
    __syncthreads();  // the staged rows are visible
    unsigned char* const q_rows = lds + kOffQ + 16 * w8 * kWRowBytes;  // this wavefront's own
    bf16x8 bq[NDS];
#pragma unroll
    for (int ds = 0; ds < NDS; ++ds)
      bq[ds] = *reinterpret_cast<const bf16x8*>(q_rows + k_lane + (wide_swz_k(col, 4 * ds + grp) << 4));

    // ---- S^T tiles: keys (rows) x queries (cols), contraction over the channels ----
    f32x4 st[NT];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const unsigned char* row = lds + ring_row(x0 + 16 * i) * kWRowBytes + k_lane;
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ds = 0; ds < NDS; ++ds)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            *reinterpret_cast<const bf16x8*>(row + (wide_swz_k(col, 4 * ds + grp) << 4)), bq[ds], acc, 0, 0, 0);
      st[i] = acc;
    }

    // ---- masked softmax over the keys; lane holds keys 16 i + 4 grp + r of query n ----
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const int klo = n0 - 64 * (NB - 1) + 16 * i;  // first key of the tile
      if (i == NT - 1 || i < i_win || klo < 0) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = klo + 4 * grp + r;
          const bool keep = key >= 0 && key <= n && key >= n - w_left;
          st[i][r] = keep ? st[i][r] : -INFINITY;
        }
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) mx = fmaxf(mx, st[i][r]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mxs = mx * scale_log2e;
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(st[i][r], scale_log2e, -mxs));  // exp2(-inf) = 0
        st[i][r] = p;
        sum += p;
      }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);

    // ---- O^T = V^T P^T: ceil(D / 16) channel tiles x NS key slabs of 32 ----
    f32x4 ot[NET];
#pragma unroll
    for (int et = 0; et < NET; ++et) ot[et] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      u32x4 pb4;
      pb4[0] = pack_bf16(st[2 * s][0], st[2 * s][1]);
      pb4[1] = pack_bf16(st[2 * s][2], st[2 * s][3]);
      if (s < NS - 1) {
        pb4[2] = pack_bf16(st[2 * s + 1][0], st[2 * s + 1][1]);
        pb4[3] = pack_bf16(st[2 * s + 1][2], st[2 * s + 1][3]);
      } else {
        pb4[2] = 0u;
        pb4[3] = 0u;
      }
      const bf16x8 bp = __builtin_bit_cast(bf16x8, pb4);
      const unsigned char* lo_rows = lds + kOffV + ring_row(x0 + 32 * s) * kWRowBytes + v_lane;
      const unsigned char* hi_rows = lds + kOffV + ring_row(s < NS - 1 ? x0 + 32 * s + 16 : 0) * kWRowBytes + v_lane;
#pragma unroll
      for (int et = 0; et < NET; ++et) {
        const int pc = wide_swz_v(vt_row, 2 * et + v_half) << 4;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(lo_rows + pc));
        s16x4 hi = {0, 0, 0, 0};
        if (s < NS - 1)
          hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(hi_rows + pc));
        const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        ot[et] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, both), bp, ot[et], 0, 0, 0);
      }
    }

    // ---- normalise; the tile goes through the wavefront's own query rows (their operand is in
    // registers, and only this wavefront rewrites them) so that every lane stores 16 bytes of a row ----
    const float inv = 1.0f / sum;
#pragma unroll
    for (int et = 0; et < NET; ++et) {
      const uint32_t w0 = pack_bf16(ot[et][0] * inv, ot[et][1] * inv);
      const uint32_t w1 = pack_bf16(ot[et][2] * inv, ot[et][3] * inv);
      *reinterpret_cast<uint2*>(q_rows + k_lane + (wide_swz_k(col, 2 * et + (grp >> 1)) << 4) + 8 * (grp & 1)) =
          make_uint2(w0, w1);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int row = 4 * it + (lane >> 4);
      const int piece = lane & 15;
      const u32x4 w4 = *reinterpret_cast<const u32x4*>(q_rows + row * kWRowBytes + (wide_swz_k(row, piece) << 4));
      if (n0 + row < L && piece < np) {
        // head rows that end inside a cache line are completed by the neighbouring head's workgroup:
        // such lines should meet in the L2 (plain store); whole lines stream past it
        u32x4* dst = reinterpret_cast<u32x4*>(o_my + (long)(n0 + row) * o_sl + 8 * piece);
        if (whole_lines) __builtin_nontemporal_store(w4, dst);
        else *dst = w4;
      }
    }

    // ---- the oldest QT blocks (and the query rows) take the next step's rows ----
    if (tile + QT < tile_end) {
      __syncthreads();  // every wavefront is done with the oldest blocks
      store_rows(oldest, q0 + kSuper, nxt, true);
      if (tile + QT * (1 + DEPTH) < tile_end) load_rows(q0 + (1 + DEPTH) * kSuper, nxt, true);  // not waited for here
    }
    q0 += kSuper;
    own = oldest;   // (own + QT) mod NBR
  };
  if constexpr (DEPTH == 1) {
    for (int tile = tile_begin; tile < tile_end; tile += QT) do_tile(tile, pre);
  } else {
    for (int tile = tile_begin; tile < tile_end; tile += 2 * QT) {
      do_tile(tile, pre);
      if (tile + QT < tile_end) do_tile(tile + QT, pre2);
    }
  }
}

// Decode step: one workgroup of four wavefronts per (b, h).  Thread t scores keys t / 4 (+ 64) over
// the 32 channels from 32 (t % 4); lane l of every wavefront owns channels 2 l, 2 l + 1 of the new
// token, of the rotation and of the output, and accumulates them over the keys congruent to its
// wavefront number mod 4.  Every load of the step is issued before anything is waited on.
template <int KB>
__global__ __launch_bounds__(256) void swa_step_wide_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ k_new, const __bf16* __restrict__ v_new,
    __bf16* __restrict__ kcache, __bf16* __restrict__ vcache, __bf16* __restrict__ o,
    const int32_t* __restrict__ cache_seqlens, int pos_host, int H, int D, int max_seqlen, long q_sb,
    long q_sh, long kn_sb, long kn_sh, long vn_sb, long vn_sh, long o_sb, long o_sh, long c_sb,
    long c_st, long c_sh, int w_left, float scale_log2e, const float* __restrict__ rope_cos,
    const float* __restrict__ rope_sin, int rope_len, int R, int interleaved) {
  constexpr int kCached = 64 * KB;
  __shared__ float s_p[kCached + 16];
  __shared__ float s_part[4][kWMaxDim];
  __shared__ __align__(16) float s_qrot[4][kWMaxDim];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bh = blockIdx.x;
  const int b = bh / H, h = bh % H;
  const int np = D >> 3;
  const bool ch_live = 2 * lane < D;       // this lane's channel pair exists
  const int ch = ch_live ? 2 * lane : 0;   // element offset of its loads
  int pos = cache_seqlens ? cache_seqlens[b] : pos_host;
  pos = __builtin_amdgcn_readfirstlane(pos);
  uint32_t* const o32 = reinterpret_cast<uint32_t*>(o + b * o_sb + h * o_sh);
  if (pos < 0 || pos >= max_seqlen || (rope_cos != nullptr && pos >= rope_len)) {
    // a device-side position outside the cache or the rotary table: the cache stays untouched and
    // the output row is NaN, so the failure shows downstream (a graph replay cannot report it)
    if (wave == 0 && ch_live) o32[lane] = 0x7FC07FC0u;
    return;
  }
  __bf16* kc = kcache + b * c_sb + h * c_sh;
  __bf16* vc = vcache + b * c_sb + h * c_sh;
  const int lo = pos - w_left > 0 ? pos - w_left : 0;
  const int ncached = pos - lo;

  // ---- issue every load of the step, unconditionally (rows past the window come from row lo,
  // pieces past the head dim from piece 0; both are masked below) ----
  const int kj = tid >> 2, kq4 = tid & 3;
  bf16x8 kx[KB][4];
#pragma unroll
  for (int g = 0; g < KB; ++g) {
    const int j = kj + 64 * g;
    const __bf16* row = kc + (long)(lo + (j < ncached ? j : 0)) * c_st;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int p = 4 * kq4 + c;
      kx[g][c] = *reinterpret_cast<const bf16x8*>(row + (p < np ? 8 * p : 0));
    }
  }
  const __bf16* qrow = q + b * q_sb + h * q_sh;
  bf16x8 qx[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int p = 4 * kq4 + c;
    qx[c] = *reinterpret_cast<const bf16x8*>(qrow + (p < np ? 8 * p : 0));
  }
  // rotary factors of this lane's channel pair at this position
  const bool do_rope = rope_cos != nullptr;
  const int half_r = R >> 1;
  const bool in_rot = do_rope && ch_live && 2 * lane < R;
  // (loaded unconditionally: without a table the reads go to the query row and are not used)
  int f0 = 0, f1 = 0, partner = lane;
  float sgn = 0.f;
  if (interleaved) {
    f0 = f1 = in_rot ? lane : 0;
  } else {
    const bool first = 2 * lane < half_r;
    f0 = in_rot ? (first ? 2 * lane : 2 * lane - half_r) : 0;
    f1 = in_rot ? f0 + 1 : 0;
    partner = in_rot ? (first ? lane + (R >> 2) : lane - (R >> 2)) : lane;
    sgn = first ? -1.0f : 1.0f;
  }
  const float* ct = do_rope ? rope_cos + (long)pos * half_r : reinterpret_cast<const float*>(q + b * q_sb + h * q_sh);
  const float* st = do_rope ? rope_sin + (long)pos * half_r : ct;
  const float cs0 = ct[f0], cs1 = ct[f1], sn0 = st[f0], sn1 = st[f1];
  constexpr int kPerWave = kCached / 4;
  uint32_t vraw[kPerWave];
#pragma unroll
  for (int u = 0; u < kPerWave; ++u) {
    const int j = 4 * u + wave;
    vraw[u] = *reinterpret_cast<const uint32_t*>(vc + (long)(lo + (j < ncached ? j : 0)) * c_st + ch);
  }
  const uint32_t kn_raw = *reinterpret_cast<const uint32_t*>(k_new + b * kn_sb + h * kn_sh + ch);
  const uint32_t vn_raw = *reinterpret_cast<const uint32_t*>(v_new + b * vn_sb + h * vn_sh + ch);
  const uint32_t ql_raw = *reinterpret_cast<const uint32_t*>(qrow + ch);
  const uint32_t live_mask = ch_live ? 0xFFFFFFFFu : 0u;
  float kn0 = bf16_bits_to_f32((kn_raw & live_mask) & 0xFFFFu), kn1 = bf16_bits_to_f32((kn_raw & live_mask) >> 16);
  const float vn0 = bf16_bits_to_f32((vn_raw & live_mask) & 0xFFFFu), vn1 = bf16_bits_to_f32((vn_raw & live_mask) >> 16);
  float ql0 = bf16_bits_to_f32((ql_raw & live_mask) & 0xFFFFu), ql1 = bf16_bits_to_f32((ql_raw & live_mask) >> 16);

  // this thread's slice of the query for the scores: 32 channels from 32 kq4 (zero past the head dim)
  float qf[32];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const bool live = 4 * kq4 + c < np;
#pragma unroll
    for (int i = 0; i < 8; ++i) qf[8 * c + i] = live ? to_f32(qx[c][i]) : 0.f;
  }
  if (do_rope) {
    // q and the new k are rotated at `pos` and rounded to bf16 like the rotated tensors of the
    // prefill; every wavefront does it for itself (lane <-> channel pair) and hands the query
    // slices round through its own LDS row
    if (interleaved) {
      const float a0 = ql0 * cs0 - ql1 * sn0, a1 = ql0 * sn0 + ql1 * cs0;
      const float b0 = kn0 * cs0 - kn1 * sn0, b1 = kn0 * sn0 + kn1 * cs0;
      if (in_rot) {
        ql0 = to_f32((__bf16)a0);
        ql1 = to_f32((__bf16)a1);
        kn0 = to_f32((__bf16)b0);
        kn1 = to_f32((__bf16)b1);
      }
    } else {
      const float pq0 = __shfl(ql0, partner, 64), pq1 = __shfl(ql1, partner, 64);
      const float pk0 = __shfl(kn0, partner, 64), pk1 = __shfl(kn1, partner, 64);
      if (in_rot) {
        ql0 = to_f32((__bf16)__builtin_fmaf(ql0, cs0, sgn * pq0 * sn0));
        ql1 = to_f32((__bf16)__builtin_fmaf(ql1, cs1, sgn * pq1 * sn1));
        kn0 = to_f32((__bf16)__builtin_fmaf(kn0, cs0, sgn * pk0 * sn0));
        kn1 = to_f32((__bf16)__builtin_fmaf(kn1, cs1, sgn * pk1 * sn1));
      }
    }
    s_qrot[wave][2 * lane] = ql0;
    s_qrot[wave][2 * lane + 1] = ql1;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const f32x4* src = reinterpret_cast<const f32x4*>(&s_qrot[wave][32 * kq4]);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const f32x4 x = src[i];
      qf[4 * i + 0] = x[0];
      qf[4 * i + 1] = x[1];
      qf[4 * i + 2] = x[2];
      qf[4 * i + 3] = x[3];
    }
  }
  if (wave == 0 && ch_live) {  // the new token joins the cache (row pos)
    *reinterpret_cast<uint32_t*>(kc + (long)pos * c_st + ch) = pack_bf16(kn0, kn1);
    *reinterpret_cast<uint32_t*>(vc + (long)pos * c_st + ch) = vn_raw;
  }

  // ---- scores ----
#pragma unroll
  for (int g = 0; g < KB; ++g) {
    float part = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int i = 0; i < 8; ++i) part = __builtin_fmaf(to_f32(kx[g][c][i]), qf[8 * c + i], part);
    part += __shfl_xor(part, 1, 64);
    part += __shfl_xor(part, 2, 64);
    if (kq4 == 0) s_p[kj + 64 * g] = kj + 64 * g < ncached ? part * scale_log2e : -INFINITY;
  }
  if (wave == 0) {
    const float self = wave_sum(ql0 * kn0 + ql1 * kn1);
    if (lane == 0) s_p[kCached] = self * scale_log2e;
  }
  __syncthreads();

  // ---- softmax over the kCached + 1 entries (every wavefront redundantly) ----
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

  // ---- output: channel pair = lane, this wavefront's keys ----
  float acc0 = wave == 0 ? p1 * vn0 : 0.f, acc1 = wave == 0 ? p1 * vn1 : 0.f;
#pragma unroll
  for (int u = 0; u < kPerWave; ++u) {
    const int j = 4 * u + wave;
    float p = __shfl(pw[u >> 4], j & 63, 64);
    p = j < ncached ? p : 0.f;
    const uint32_t raw = vraw[u] & (j < ncached ? live_mask : 0u);
    acc0 = __builtin_fmaf(p, bf16_bits_to_f32(raw & 0xFFFFu), acc0);
    acc1 = __builtin_fmaf(p, bf16_bits_to_f32(raw >> 16), acc1);
  }
  s_part[wave][2 * lane] = acc0;
  s_part[wave][2 * lane + 1] = acc1;
  __syncthreads();
  if (wave == 0 && ch_live) {
    const float t0 = s_part[0][2 * lane] + s_part[1][2 * lane] + s_part[2][2 * lane] + s_part[3][2 * lane];
    const float t1 = s_part[0][2 * lane + 1] + s_part[1][2 * lane + 1] + s_part[2][2 * lane + 1] + s_part[3][2 * lane + 1];
    o32[lane] = pack_bf16(t0 / denom, t1 / denom);
  }
}

static bool wide_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

constexpr int kWideMaxDevices = 64;
static std::atomic<bool> g_wide_lds_allowed[kWideMaxDevices][3 /*RMODE*/][3 /*NB 2, NB 3, NB 3 two tiles*/][2 /*NDS / 2 - 1*/];

// shared checks of the rotary arguments; returns the layout code or -1 with the error set
static int wide_rope_mode(const char* who, const float* rope_cos, const float* rope_sin, int64_t rotary_dim,
                          int rotary_interleaved, int64_t D) {
  if ((rope_cos == nullptr) != (rope_sin == nullptr)) {
    set_error("%s: rotary tables must be given together", who);
    return -1;
  }
  if (rope_cos == nullptr) return kRopeNone;
  if (rotary_dim <= 0 || rotary_dim > D || rotary_dim % 16 != 0) {
    set_error("%s: rotary_dim %ld unsupported (a positive multiple of 16, at most the head dim %ld)", who,
              (long)rotary_dim, (long)D);
    return -1;
  }
  if (!wide_aligned16(rope_cos) || !wide_aligned16(rope_sin)) {
    set_error("%s: rotary tables must be 16-byte aligned", who);
    return -1;
  }
  return rotary_interleaved ? kRopeInterleaved : kRopeHalf;
}

}  // namespace based

extern "C" BASED_API int based_swa_prefill_wide(const void* q, const void* k, const void* v, void* o, int64_t B,
                                                int64_t H, int64_t L, int64_t D, int64_t q_sb, int64_t q_sl,
                                                int64_t q_sh, int64_t k_sb, int64_t k_sl, int64_t k_sh, int64_t v_sb,
                                                int64_t v_sl, int64_t v_sh, int64_t o_sb, int64_t o_sl, int64_t o_sh,
                                                int w_left, float scale, const float* rope_cos,
                                                const float* rope_sin, int64_t rope_len, int64_t rotary_dim,
                                                int rotary_interleaved, void* kcache_out, void* vcache_out,
                                                int64_t c_sb, int64_t c_st, int64_t c_sh, int64_t max_seqlen,
                                                int io_dtype, void* stream) {
  using namespace based;
  BASED_REQUIRE(q && k && v && o, BASED_ERR_ARG, "swa_prefill_wide: null pointer argument");
  BASED_REQUIRE(D >= 8 && D <= kWMaxDim && D % 8 == 0, BASED_ERR_SHAPE,
                "swa_prefill_wide: head dim %ld unsupported (multiples of 8 up to %d)", (long)D, kWMaxDim);
  const int rmode = wide_rope_mode("swa_prefill_wide", rope_cos, rope_sin, rotary_dim, rotary_interleaved, D);
  if (rmode < 0) return BASED_ERR_ARG;
  if (rmode != kRopeNone)
    BASED_REQUIRE(rope_len >= L, BASED_ERR_ARG, "swa_prefill_wide: rotary tables hold %ld positions, need %ld",
                  (long)rope_len, (long)L);
  BASED_REQUIRE((kcache_out == nullptr) == (vcache_out == nullptr), BASED_ERR_ARG,
                "swa_prefill_wide: cache outputs must be given together");
  if (kcache_out) {
    BASED_REQUIRE(L <= max_seqlen, BASED_ERR_SHAPE, "swa_prefill_wide: %ld tokens do not fit a cache of %ld rows",
                  (long)L, (long)max_seqlen);
    BASED_REQUIRE(c_sb % 8 == 0 && c_st % 8 == 0 && c_sh % 8 == 0, BASED_ERR_ALIGN,
                  "swa_prefill_wide: cache strides must be multiples of 8 elements");
    BASED_REQUIRE(wide_aligned16(kcache_out) && wide_aligned16(vcache_out), BASED_ERR_ALIGN,
                  "swa_prefill_wide: caches must be 16-byte aligned");
  }
  BASED_REQUIRE(B >= 0 && H > 0 && L >= 0, BASED_ERR_ARG, "swa_prefill_wide: bad sizes");
  BASED_REQUIRE(io_dtype == BASED_BF16, BASED_ERR_DTYPE, "swa_prefill_wide: only bf16 is supported");
  BASED_REQUIRE(w_left >= 0 && w_left <= 128, BASED_ERR_SHAPE, "swa_prefill_wide: left window %d unsupported (0..128)",
                w_left);
  BASED_REQUIRE(H < 65536 && B < 65536 && L < (1ll << 31) - 64, BASED_ERR_SHAPE, "swa_prefill_wide: grid too large");
  const int64_t strides[] = {q_sb, q_sl, q_sh, k_sb, k_sl, k_sh, v_sb, v_sl, v_sh, o_sb, o_sl, o_sh};
  for (int64_t s : strides)
    BASED_REQUIRE(s % 8 == 0, BASED_ERR_ALIGN, "swa_prefill_wide: strides must be multiples of 8 elements");
  BASED_REQUIRE(wide_aligned16(q) && wide_aligned16(k) && wide_aligned16(v) && wide_aligned16(o), BASED_ERR_ALIGN,
                "swa_prefill_wide: tensors must be 16-byte aligned");
  if (B == 0 || L == 0) return BASED_OK;
  const int64_t n_tiles = (L + kWQTile - 1) / kWQTile;
  BASED_REQUIRE(B * H * n_tiles < (1ll << 31), BASED_ERR_SHAPE, "swa_prefill_wide: grid too large");
  const int nb = w_left > 64 ? 3 : 2;
  // the three-block window: two tiles side by side per workgroup (a sequence of one tile has nothing for the second)
  const int qt = nb == 3 && n_tiles > 1 ? 2 : 1;
  // runs of consecutive tiles, as long as still gives every resident slot one run: 256 compute
  // units x the workgroups whose LDS fits one (80 KB: two; 112 KB and 160 KB: one)
  const int64_t slots = 256 * (nb == 3 ? 1 : 2);
  int64_t want_runs = slots / (B * H);
  want_runs = want_runs < 1 ? 1 : (want_runs > n_tiles ? n_tiles : want_runs);
  int64_t run_tiles = (n_tiles + want_runs - 1) / want_runs;
  run_tiles = (run_tiles + qt - 1) / qt * qt;
  const int64_t runs_per_seq = (n_tiles + run_tiles - 1) / run_tiles;
  dim3 grid((unsigned)(B * H * runs_per_seq)), block(256 * qt);
  using Kern = void (*)(const __bf16*, const __bf16*, const __bf16*, __bf16*, int, int, int, int, int, long, long, long,
                        long, long, long, long, long, long, long, long, long, int, float, const float*, const float*, int,
                        __bf16*, __bf16*, long, long, long);
  // head dims up to 64 contract in two steps of 32 channels, up to 128 in four
  static const Kern kerns[3][3][2] = {
      {{swa_prefill_wide_kernel<kRopeNone, 2, 2, 1>, swa_prefill_wide_kernel<kRopeNone, 2, 4, 1>},
       {swa_prefill_wide_kernel<kRopeNone, 3, 2, 1>, swa_prefill_wide_kernel<kRopeNone, 3, 4, 1>},
       {swa_prefill_wide_kernel<kRopeNone, 3, 2, 2>, swa_prefill_wide_kernel<kRopeNone, 3, 4, 2>}},
      {{swa_prefill_wide_kernel<kRopeHalf, 2, 2, 1>, swa_prefill_wide_kernel<kRopeHalf, 2, 4, 1>},
       {swa_prefill_wide_kernel<kRopeHalf, 3, 2, 1>, swa_prefill_wide_kernel<kRopeHalf, 3, 4, 1>},
       {swa_prefill_wide_kernel<kRopeHalf, 3, 2, 2>, swa_prefill_wide_kernel<kRopeHalf, 3, 4, 2>}},
      {{swa_prefill_wide_kernel<kRopeInterleaved, 2, 2, 1>, swa_prefill_wide_kernel<kRopeInterleaved, 2, 4, 1>},
       {swa_prefill_wide_kernel<kRopeInterleaved, 3, 2, 1>, swa_prefill_wide_kernel<kRopeInterleaved, 3, 4, 1>},
       {swa_prefill_wide_kernel<kRopeInterleaved, 3, 2, 2>, swa_prefill_wide_kernel<kRopeInterleaved, 3, 4, 2>}}};
  const int wide = D > 64 ? 1 : 0;
  const int variant = nb - 2 + (qt - 1);
  const Kern kern = kerns[rmode][variant][wide];
  const size_t lds = (size_t)wide_lds_bytes(nb, qt);
  {
    int dev = 0;
    BASED_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kWideMaxDevices, BASED_ERR_LAUNCH,
                  "swa_prefill_wide: cannot identify the current device");
    std::atomic<bool>& allowed = g_wide_lds_allowed[dev][rmode][variant][wide];
    if (!allowed.load(std::memory_order_acquire)) {  // more than 64 KB of LDS has to be asked for once per device
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      BASED_REQUIRE(e == hipSuccess, BASED_ERR_LAUNCH, "swa_prefill_wide: cannot raise the LDS limit to %zu bytes: %s",
                    lds, hipGetErrorString(e));
      allowed.store(true, std::memory_order_release);
    }
  }
  hipLaunchKernelGGL(kern, grid, block, lds, static_cast<hipStream_t>(stream), (const __bf16*)q, (const __bf16*)k,
                     (const __bf16*)v, (__bf16*)o, (int)H, (int)L, (int)D, (int)n_tiles, (int)run_tiles, q_sb, q_sl, q_sh,
                     k_sb, k_sl, k_sh, v_sb, v_sl, v_sh, o_sb, o_sl, o_sh, w_left, scale * 1.4426950408889634f, rope_cos,
                     rope_sin, (int)rotary_dim, (__bf16*)kcache_out, (__bf16*)vcache_out, c_sb, c_st, c_sh);
  return check_launch("swa_prefill_wide");
}

extern "C" BASED_API int based_swa_step_wide(const void* q, const void* k_new, const void* v_new, void* kcache,
                                             void* vcache, void* o, const int32_t* cache_seqlens, int64_t pos_host,
                                             int64_t B, int64_t H, int64_t D, int64_t max_seqlen, int64_t q_sb,
                                             int64_t q_sh, int64_t kn_sb, int64_t kn_sh, int64_t vn_sb, int64_t vn_sh,
                                             int64_t o_sb, int64_t o_sh, int64_t c_sb, int64_t c_st, int64_t c_sh,
                                             int w_left, float scale, const float* rope_cos, const float* rope_sin,
                                             int64_t rope_len, int64_t rotary_dim, int rotary_interleaved,
                                             int io_dtype, void* stream) {
  using namespace based;
  BASED_REQUIRE(q && k_new && v_new && kcache && vcache && o, BASED_ERR_ARG, "swa_step_wide: null pointer argument");
  BASED_REQUIRE(D >= 8 && D <= kWMaxDim && D % 8 == 0, BASED_ERR_SHAPE,
                "swa_step_wide: head dim %ld unsupported (multiples of 8 up to %d)", (long)D, kWMaxDim);
  const int rmode = wide_rope_mode("swa_step_wide", rope_cos, rope_sin, rotary_dim, rotary_interleaved, D);
  if (rmode < 0) return BASED_ERR_ARG;
  if (rmode != kRopeNone) {
    BASED_REQUIRE(rope_len > 0 && rope_len < (1ll << 31), BASED_ERR_ARG, "swa_step_wide: bad rotary table length");
    if (!cache_seqlens)
      BASED_REQUIRE(pos_host < rope_len, BASED_ERR_ARG, "swa_step_wide: position %ld beyond the rotary table (%ld rows)",
                    (long)pos_host, (long)rope_len);
  }
  BASED_REQUIRE(B >= 0 && H > 0 && max_seqlen > 0, BASED_ERR_ARG, "swa_step_wide: bad sizes");
  BASED_REQUIRE(io_dtype == BASED_BF16, BASED_ERR_DTYPE, "swa_step_wide: only bf16 is supported");
  BASED_REQUIRE(w_left >= 0 && w_left <= 128, BASED_ERR_SHAPE, "swa_step_wide: left window %d unsupported (0..128)",
                w_left);
  BASED_REQUIRE(max_seqlen < (1ll << 31) && B * H < (1ll << 31), BASED_ERR_SHAPE, "swa_step_wide: sizes too large");
  if (!cache_seqlens)
    BASED_REQUIRE(pos_host >= 0 && pos_host < max_seqlen, BASED_ERR_ARG,
                  "swa_step_wide: position %ld outside the cache (max_seqlen %ld)", (long)pos_host, (long)max_seqlen);
  const int64_t strides[] = {q_sb, q_sh, kn_sb, kn_sh, vn_sb, vn_sh, o_sb, o_sh, c_sb, c_st, c_sh};
  for (int64_t s : strides)
    BASED_REQUIRE(s % 8 == 0, BASED_ERR_ALIGN, "swa_step_wide: strides must be multiples of 8 elements");
  BASED_REQUIRE(wide_aligned16(kcache) && wide_aligned16(vcache) && wide_aligned16(q) && wide_aligned16(k_new) &&
                    wide_aligned16(v_new) && wide_aligned16(o),
                BASED_ERR_ALIGN, "swa_step_wide: tensors must be 16-byte aligned");
  if (B == 0) return BASED_OK;
  hipLaunchKernelGGL(w_left > 64 ? swa_step_wide_kernel<2> : swa_step_wide_kernel<1>, dim3((unsigned)(B * H)), dim3(256),
                     0, static_cast<hipStream_t>(stream), (const __bf16*)q, (const __bf16*)k_new, (const __bf16*)v_new,
                     (__bf16*)kcache, (__bf16*)vcache, (__bf16*)o, cache_seqlens, (int)pos_host, (int)H, (int)D,
                     (int)max_seqlen, q_sb, q_sh, kn_sb, kn_sh, vn_sb, vn_sh, o_sb, o_sh, c_sb, c_st, c_sh, w_left,
                     scale * 1.4426950408889634f, rope_cos, rope_sin, (int)rope_len, (int)rotary_dim, rotary_interleaved);
  return check_launch("swa_step_wide");
}
