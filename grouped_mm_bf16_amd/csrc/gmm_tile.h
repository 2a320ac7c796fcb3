// One 256 x 256 output tile of C = A * B on gfx950: C++ wrapper around the generated assembly
// (gmm_tile_asm.inc, made by gen_tile_asm.py).  The wrapper turns a tile description into the
// per-lane offsets and the scalars the assembly expects in fixed registers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int gmm_v4i __attribute__((ext_vector_type(4)));
typedef int gmm_v8i __attribute__((ext_vector_type(8)));
typedef int gmm_v2i __attribute__((ext_vector_type(2)));

struct GmmTileRegs {
  gmm_v8i voa_head, vob_head;  // copy offsets of K tile 0 (first/last chunk masks applied)
  gmm_v8i voa, vob;            // copy offsets of a full K tile
  gmm_v8i voa_tail, vob_tail;  // copy offsets of the last K tile
  gmm_v4i ra_addr, rb_addr;    // LDS fragment read addresses
  gmm_v4i epi;                 // epilogue: per-lane addresses (see gen_tile_asm.py)
  gmm_v2i epi2;                // bf16 epilogue: store offset of the lane's chunk whatever its validity; mask of
                               // its valid elements when only some of them are (a group boundary inside it)
  gmm_v2i touch;               // L2 prefetch: byte offset of the cache line this lane touches in K tile 0 of A, of B (or out of range)
  gmm_v4i fix;                 // LDS addresses of this thread's row in the first / last k chunk (A, A, B, B)
  gmm_v8i masks;               // keep-masks of the first and of the last 16-byte k chunk
  gmm_v4i rsrc_a, rsrc_b, rsrc_c;
  gmm_v8i scal;                // nk, a_step, b_step, lds_base, row_cnt, c_step, (unused), wave | flags << 8
};

// TM = MFMA block rows per wave: the tile is 64 * TM rows (256, 128 or 64) by 256 columns.
// F16 = 1: A, B and a 16-bit output are fp16 instead of bf16 (same layouts, other MFMA and conversion).
// B_NT = 1 (128- and 64-row tiles): B is copied with the non-temporal hint, for a tile that is the only
// reader of its B panel (it then does not push panels that other tiles share out of the L2).
// ACT = 2: the tile is a partial sum (a part of a tile cut along K): fp32, stored through to memory at
// device scope (sc1), so that a workgroup on another XCD can read it without anybody flushing an L2.
// ACT = 1: SwiGLU epilogue.  Of every 128 columns of the product the first 64 are gates g and the last 64
// their partners u; the tile stores silu(g) * u: 128 columns of a 16-bit output per 256-column tile.
template <int A_TR, int B_TR, int OUT_F32, int TM, int F16, int B_NT, int ACT>
__device__ __forceinline__ void gmm_tile_asm(GmmTileRegs& r);

#include "gmm_tile_asm.inc"

constexpr int GMM_TILE_M = 256, GMM_TILE_N = 256, GMM_TILE_K = 64;
constexpr unsigned GMM_OOB = 0x80000000u;

// Pipeline depth and LDS layout of a tile of 64 * TM rows: `stages` buffers of A from offset 0, then as
// many of B.  The 256-row tile has two buffers (LDS is full); the shorter ones have
// GMM_TILE_STAGES_SHORT, and with three their A buffers shrink to the rows they hold.
template <int A_TR, int TM>
struct GmmTileLayout {
  static constexpr int stages = TM == 4 ? 2 : GMM_TILE_STAGES_SHORT;
  static constexpr int a_stage = A_TR ? GMM_TILE_TR_STAGE : (stages == 3 ? 64 * TM * 128 : GMM_TILE_KC_STAGE);
  static constexpr int b_base = stages * a_stage;
};

// LDS bytes one workgroup needs for tiles of 64 * TM rows: the pipeline buffers, or the staging area of
// the bf16 epilogue (one padded row of 256 columns per tile row).
template <int A_TR, int B_TR, int TM>
constexpr int gmm_tile_lds_bytes() {
  using L = GmmTileLayout<A_TR, TM>;
  constexpr int pipe = L::b_base + L::stages * (B_TR ? GMM_TILE_TR_STAGE : GMM_TILE_KC_STAGE);
  // staging of the epilogue: one padded row of 256 columns per tile row (16-bit output), or 32 rows of
  // 128 fp32 columns per wave and pass; both are below the pipeline buffers of every tile height
  constexpr int staging16 = 64 * TM * 2 * GMM_TILE_PITCH, staging32 = 4 * 32 * GMM_TILE_PITCH32;
  constexpr int staging = staging16 > staging32 ? staging16 : staging32;
  return pipe > staging ? pipe : staging;
}

__device__ __forceinline__ gmm_v4i gmm_make_rsrc(const void* p, long long bytes) {
  const unsigned long long a = (unsigned long long)p;
  if (bytes < 0) bytes = 0;
  if (bytes > 0x7fffffffLL) bytes = 0x7fffffffLL;
  gmm_v4i r = {__builtin_amdgcn_readfirstlane((int)(unsigned)a),
               __builtin_amdgcn_readfirstlane((int)(unsigned)((a >> 32) & 0xffffu)),
               __builtin_amdgcn_readfirstlane((int)bytes), 0x00020000};
  return r;
}

__device__ __forceinline__ int gmm_swz(int row) { return (row >> 1) & 7; }

// One operand of a tile.  `base` points at element (row 0 of the tile, k_begin) of the operand;
// `ld` is the leading dimension in elements; `bytes` is the distance from `base` to the end of the
// operand's storage (reads past it return zero).
struct GmmOperand {
  const uint16_t* base;
  int ld;
  long long bytes;
  // Row gather (first operand, contiguous along K only): tile row r reads row gather[r] of the matrix at
  // `base` (which then points at row 0), for r < gather_n; other rows, and indices outside [0, src_rows),
  // read as zeros.  Null: tile row r is row r from `base`.
  const int32_t* gather = nullptr;
  int gather_n = 0, src_rows = 0;
};

// Description of one tile for the assembly.  klen = number of k elements from k_begin that count.
struct GmmTileDesc {
  GmmOperand a, b;
  void* c;               // element (m0, n0) of the output
  int ldc;
  long long c_bytes;     // from c to the end of the output storage
  int klen;              // k elements from k_begin that count ...
  int khead;             // ... of which the first khead are before the group's range (0..7) and read as zero
  int row_rel0;          // m0 - m_lo   (may be negative: rows before m_lo are not stored)
  int row_cnt;           // m_hi - m_lo
  int col_lo, col_hi;    // columns [col_lo, col_hi) of the tile are stored (relative to n0; with the SwiGLU
                         // epilogue: output columns relative to n0 / 2)
  int share, sharers;    // L2 prefetch of B: this tile touches share number `share` of `sharers` (0: none)
};

// NI = copy instructions per wave and K tile for this operand (8 for 256 rows, 2 per 64 rows).
// klen, khead and nk are the same for all lanes: whether the first / last K tile is a whole one is a
// scalar branch, and only partial ones pay for the per-lane selects.
template <int TR, int NI>
__device__ __forceinline__ void gmm_copy_offsets(int lane, int wave, const GmmOperand& op, int klen, int khead, int nk,
                                                 gmm_v8i& head, gmm_v8i& full, gmm_v8i& tail) {
  const int ld = op.ld;
  int kk[8];
  // gathered rows: all index loads first (one wait for the lot), then the range checks
  int src[8];
  if (!TR && op.gather) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int row = wave * (NI * 8) + i * 8 + (lane >> 3);
      src[i] = op.gather[row < op.gather_n ? row : 0];
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int row = wave * (NI * 8) + i * 8 + (lane >> 3);
      if (row >= op.gather_n || src[i] >= op.src_rows) src[i] = -1;
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    if (i >= NI) { kk[i] = 0; full[i] = (int)GMM_OOB; continue; }
    if (!TR) {
      const int row = wave * (NI * 8) + i * 8 + (lane >> 3);
      const int c = (lane & 7) ^ gmm_swz(row);
      kk[i] = c * 8;
      const int r = op.gather ? src[i] : row;
      full[i] = r >= 0 ? r * ld * 2 + c * 16 : (int)GMM_OOB;
    } else {
      const int blk = wave * 8 + i;
      kk[i] = 8 * (blk >> 2) + (blk & 3) + 4 * (lane >> 5);
      full[i] = kk[i] * ld * 2 + (lane & 31) * 16;
    }
  }
  head = full;
  tail = full;
  if (!(khead == 0 && klen >= GMM_TILE_K)) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      // whole k rows before the range are skipped (transposed layout); inside a chunk the fix-up masks them
      const bool before = TR && kk[i] < khead;
      head[i] = (kk[i] < klen && !before) ? full[i] : (int)GMM_OOB;
    }
  }
  if (!(klen > 0 && (klen & (GMM_TILE_K - 1)) == 0 && !(khead != 0 && nk == 1))) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const bool before = TR && kk[i] < khead;
      tail[i] = ((nk - 1) * GMM_TILE_K + kk[i] < klen && !(before && nk == 1)) ? full[i] : (int)GMM_OOB;
    }
  }
}

template <int A_TR, int B_TR, int OUT_F32, int TM = 4, int F16 = 0, int B_NT = 0, int ACT = 0>
__device__ __forceinline__ void gmm_tile_compute(const GmmTileDesc& t, unsigned lds_base, int lane, int wave) {
  static_assert(TM == 4 || !A_TR, "short tiles exist for a K-contiguous A only");
  static_assert(ACT != 1 || (!A_TR && !OUT_F32), "the SwiGLU epilogue: K-contiguous A, 16-bit output");
  static_assert(ACT != 2 || (OUT_F32 && !B_NT), "partial tiles are fp32");
  constexpr int WROWS = 32 * TM;  // rows of the tile per wave row
  constexpr int B_BASE = GmmTileLayout<A_TR, TM>::b_base;
  const int wm = wave & 1, wn = wave >> 1;
  const int nk = (t.klen + GMM_TILE_K - 1) / GMM_TILE_K;
  GmmTileRegs r;
  gmm_copy_offsets<A_TR, 2 * TM>(lane, wave, t.a, t.klen, t.khead, nk, r.voa_head, r.voa, r.voa_tail);
  gmm_copy_offsets<B_TR, 8>(lane, wave, t.b, t.klen, t.khead, nk, r.vob_head, r.vob, r.vob_tail);
  // Fragment read addresses.  An MFMA fragment is 16 rows (or columns) x 32 k: lane l holds row l % 16,
  // k 8 (l / 16) .. + 7.  K-contiguous operand: one ds_read_b128 of chunk 4 sp + l / 16 of the lane's row
  // (sp = k half of the K tile; one address per half, 16-row blocks are immediate offsets).  Transposed
  // layout: two ds_read_b64_tr_b16, each a 4 (k) x 16 (rows) block whose 16 lanes address 4 consecutive
  // rows of k row ii / 4; k rows 8 q .. 8 q + 3 are the first rows of LDS blocks 4 q .. 4 q + 3 (k halves,
  // 16-row blocks and the second four k rows are immediate offsets).
  const int q = lane >> 4, ii = lane & 15;
  r.ra_addr = gmm_v4i{0, 0, 0, 0};
  r.rb_addr = gmm_v4i{0, 0, 0, 0};
#pragma unroll
  for (int sp = 0; sp < 2; ++sp) {
    const int chunk = 4 * sp + q;
    if (!A_TR) {
      const int row = wm * WROWS + ii;
      r.ra_addr[sp] = lds_base + row * 128 + ((chunk ^ gmm_swz(row)) << 4);
    } else if (sp == 0) {
      r.ra_addr[0] = lds_base + (4 * q + (ii >> 2)) * GMM_TILE_TR_BLOCK + (wm * 128 + 4 * (ii & 3)) * 2;
    }
    if (!B_TR) {
      const int row = wn * 128 + ii;
      r.rb_addr[sp] = lds_base + B_BASE + row * 128 + ((chunk ^ gmm_swz(row)) << 4);
    } else if (sp == 0) {
      r.rb_addr[0] = lds_base + B_BASE + (4 * q + (ii >> 2)) * GMM_TILE_TR_BLOCK + (wn * 128 + 4 * (ii & 3)) * 2;
    }
  }
  // Epilogue: the wave stages its block in LDS and reads it back row by row, 16 bytes per lane (see
  // gen_tile_asm.py).  ESZ bytes per element: a lane's chunk is NEL = 16 / ESZ columns, a row of the wave's
  // 128 columns takes LPR lanes, a read-back instruction covers 64 / LPR rows.
  constexpr int WCOLS = ACT == 1 ? 64 : 128;                   // output columns of a wave
  constexpr int ESZ = OUT_F32 ? 4 : 2, NEL = 16 / ESZ, LPR = WCOLS / NEL;
  constexpr int EPITCH = OUT_F32 ? GMM_TILE_PITCH32 : (ACT == 1 ? GMM_TILE_PITCH_ACT : GMM_TILE_PITCH);
  constexpr int STAGE_ROWS = OUT_F32 ? 32 : WROWS;        // rows a wave stages per pass
  int partial = 0;
  {
    const int row_t = wm * WROWS + lane / LPR, col_t = wn * WCOLS + (lane % LPR) * NEL;
    const unsigned stage = lds_base + wave * (STAGE_ROWS * EPITCH);
    r.epi[0] = stage + (lane & 15) * EPITCH + 4 * ESZ * (lane >> 4);        // write: row lane % 16, columns 4 (lane / 16) ..
    r.epi[1] = stage + (lane / LPR) * EPITCH + (lane % LPR) * 16;           // read: row lane / LPR, chunk lane % LPR
    // the lane's columns: all valid -> one 16-byte store; some valid (a group boundary inside the chunk)
    // -> element stores under the mask; none -> nothing
    int mask = 0;
#pragma unroll
    for (int e = 0; e < NEL; ++e) mask |= (col_t + e >= t.col_lo && col_t + e < t.col_hi) ? (1 << e) : 0;
    constexpr int FULL = (1 << NEL) - 1;
    const int off = (row_t * t.ldc + col_t) * ESZ;
    r.epi[2] = mask == FULL ? off : (int)GMM_OOB;
    r.epi[3] = t.row_rel0 + row_t;
    r.epi2[0] = off;
    r.epi2[1] = mask == FULL ? 0 : mask;
    partial = ((t.col_lo | t.col_hi) & (NEL - 1)) ? 1 : 0;
  }
  // L2 prefetch touches of B.  A K tile of B is 256 cache lines of 128 bytes: one per row when B is
  // contiguous along K, else four per k row (64 k rows of 512 bytes).  The tile rows of a band run at the
  // same time on one XCD and read the same B panel: each of the `sharers` tiles touches its own share of the
  // lines, a quarter of it per wave, so every line is requested once, early, and the copies of all sharers hit.
  {
    int off_b = (int)GMM_OOB;
    if (t.sharers > 0) {
      const int per_tile = (256 + t.sharers - 1) / t.sharers, per_wave = (per_tile + 3) >> 2;
      const int idx = wave * per_wave + lane, line = t.share * per_tile + idx;
      if (lane < per_wave && idx < per_tile && line < 256)
        off_b = B_TR ? (line >> 2) * t.b.ld * 2 + (line & 3) * 128 : line * t.b.ld * 2;
    }
    r.touch[0] = (int)GMM_OOB;
    r.touch[1] = off_b;
  }
  const int c_step = (64 / LPR) * t.ldc * ESZ;
  const int n_valid = 0;
  r.rsrc_a = gmm_make_rsrc(t.a.base, t.a.bytes);
  r.rsrc_b = gmm_make_rsrc(t.b.base, t.b.bytes);
  r.rsrc_c = gmm_make_rsrc(t.c, t.c_bytes);
  const int a_step = A_TR ? GMM_TILE_K * t.a.ld * 2 : GMM_TILE_K * 2;
  const int b_step = B_TR ? GMM_TILE_K * t.b.ld * 2 : GMM_TILE_K * 2;
  // partial first / last chunk of the k range (jagged contraction with an operand contiguous along K)
  const int ktail = t.klen & 7;
  int flags = 0;
  if (!(A_TR && B_TR)) flags = (t.khead ? 1 : 0) | (ktail ? 2 : 0);
  flags |= partial << 2;
  {
    // one row of each operand tile per thread (A tiles shorter than 256 rows: several threads per row,
    // all writing the same masked value)
    const int row = wave * 64 + lane, row_a = row % (64 * TM);
    const int c_last = ((t.klen - 1) & (GMM_TILE_K - 1)) >> 3;
    r.fix[0] = lds_base + row_a * 128 + ((0 ^ gmm_swz(row_a)) << 4);
    r.fix[1] = lds_base + row_a * 128 + ((c_last ^ gmm_swz(row_a)) << 4);
    r.fix[2] = lds_base + B_BASE + row * 128 + ((0 ^ gmm_swz(row)) << 4);
    r.fix[3] = lds_base + B_BASE + row * 128 + ((c_last ^ gmm_swz(row)) << 4);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const unsigned h0 = (2 * w >= t.khead) ? 0x0000ffffu : 0u, h1 = (2 * w + 1 >= t.khead) ? 0xffff0000u : 0u;
      const unsigned t0 = (2 * w < ktail) ? 0x0000ffffu : 0u, t1 = (2 * w + 1 < ktail) ? 0xffff0000u : 0u;
      r.masks[w] = __builtin_amdgcn_readfirstlane((int)(h0 | h1));
      r.masks[4 + w] = __builtin_amdgcn_readfirstlane((int)(t0 | t1));
    }
  }
  const int sc[8] = {nk, a_step, b_step, (int)lds_base, t.row_cnt, c_step, n_valid, wave | (flags << 8)};
#pragma unroll
  for (int i = 0; i < 8; ++i) r.scal[i] = __builtin_amdgcn_readfirstlane(sc[i]);
  gmm_tile_asm<A_TR, B_TR, OUT_F32, TM, F16, B_NT, ACT>(r);
}
