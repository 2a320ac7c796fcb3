// Tile scheduler shared by host and device.
//
// A grouped matrix multiply is a list of independent GEMM problems, one per
// group, that differ only along one "jagged" dimension (rows for 2D x 3D,
// columns for 3D x 2D, the contraction for 2D x 2D, none for 3D x 3D).  The
// group boundaries live in device memory (`offs`, int32 end offsets), so the
// number of output tiles is unknown to the host.  Every workgroup therefore
// builds the same table on its own: per-group tile counts, their exclusive
// prefix sum, and a decode from a linear tile id to (group, tile row, tile
// column).  The functions here are that logic; they compile for the host too,
// so the CPU tests can enumerate tiles exactly as the kernels do.
//
// Semantics followed (reference tree): the group that owns index i is the first
// g with offs[g] > i (grouped_mm_bf16/kernels.py:162-172); empty groups own
// nothing in 2D x 3D / 3D x 2D but still produce an all-zero slab in 2D x 2D
// (kernels.py:276-301).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define GMM_HD __host__ __device__ __forceinline__
#else
#define GMM_HD inline
#endif

enum GmmJag : int32_t { GMM_JAG_NONE = 0, GMM_JAG_M = 1, GMM_JAG_N = 2, GMM_JAG_K = 3 };

constexpr int GMM_MAX_GROUPS = 1024;  // offs.numel() < 1024 is enforced by the host layer
constexpr int GMM_BAND = 8;           // tile rows per band in the within-group tile order

// Everything a kernel needs to know about one call.  Strides are in elements.
struct GmmParams {
  const void* a;
  const void* b;
  void* c;
  const int32_t* offs;
  int32_t G;        // number of groups (batch size for 3D x 3D)
  int32_t jag;      // GmmJag
  int32_t M, N, K;  // full extents; the jagged one is the total over groups
  int32_t align;    // tile origins along the jagged dimension are rounded down to this
  int64_t a_sg, a_sm, a_sk;
  int64_t b_sg, b_sk, b_sn;
  int64_t c_sg, c_sm, c_sn;
  int32_t xcd_remap;  // 1: renumber tiles so that each XCD works on a compact block
  int32_t num_wg;     // persistent grid size
  int32_t tall;       // tile list with several heights: rows of a "tall" tile (256 or 128) ...
  int32_t shrt;       // ... and of the shortest tile for group remainders (64), or 0: tall tiles only
  // Row gather for the first operand (jagged rows only): row r of the product reads row gather[r] of `a`
  // (which then has `a_rows` rows); null: row r reads row r.
  const int32_t* gather;
  int32_t a_rows;
  // 1: SwiGLU epilogue (assembly tile, jagged rows, 16-bit output): `c` has N / 2 columns, see gmm_tile.h
  int32_t act;
  // Split of the last, partly filled round of the launch along K (assembly tile; see gmm_tail_split): fp32
  // partial tiles go to `ws` (GMM_WS_HEADER bytes of arrival counters that are zero between launches, then
  // `ws_parts` slots of GMM_WS_SLOT bytes); null / 0: no split.
  void* ws;
  int32_t ws_parts;
  // Launch order of tiles of different heights.  0: all tall tiles of all groups, then all remainder tiles.
  // 1: group by group, a group's remainder tiles right after its tall tiles, while the group's second
  // operand is still in the Infinity Cache.
  int32_t group_major;
};

constexpr int GMM_WS_HEADER = 4096;          // 1024 int32: arrival counters, one per tile of the split round, ...
constexpr int GMM_WS_SLOT = 256 * 256 * 4;   // one fp32 partial tile
constexpr int GMM_SPLIT_MAX = 8;             // most parts a tile is cut into
constexpr int GMM_SPLIT_PART_MIN = 32;       // fewest K tiles (of 64) of a part
constexpr int GMM_SPLIT_PART_COST = 20;      // what a part costs beyond its K tiles, in K tiles (gmm_tail_split):
                                             // measured, a round of 56 tiles of 64 K tiles cut four ways takes as long as uncut
constexpr int GMM_WS_TICKET = 1020;          // header words beyond the arrival counters: next part to hand out,
constexpr int GMM_WS_EXITED = 1021;          // workgroups that have left the ticket loop

GMM_HD int gmm_cdiv(int a, int b) { return (a + b - 1) / b; }
GMM_HD int gmm_min(int a, int b) { return a < b ? a : b; }
GMM_HD int gmm_max(int a, int b) { return a > b ? a : b; }

// A persistent launch deals `total` tiles to W workgroups round by round; the last round holds
// tail = total % W tiles and leaves W - tail workgroups idle for a whole tile.  When the workspace allows,
// every tile of that round is cut along K into S parts (its K tiles split evenly) that any free workgroup
// takes from a ticket counter; each part stores an fp32 partial tile, and the part that arrives last adds the
// partials in part order (the sum does not depend on timing) and stores the output.  Returns S (1: no
// split): the S that makes the round shortest when a part costs its K tiles plus GMM_SPLIT_PART_COST (its
// prologue, the fp32 store of the partial tile and its share of the reduction, in K tiles) and tail * S parts
// take ceil(tail * S / W) turns; at most GMM_SPLIT_MAX parts per tile, as the workspace allows, none shorter
// than GMM_SPLIT_PART_MIN K tiles, and only if the round gets at least a fifth shorter.  nk = K tiles per tile
// (the same for every tile: not for a jagged contraction).
GMM_HD int gmm_tail_split(int total, int W, int nk, int max_parts) {
  const int tail = total % W;
  if (tail == 0 || tail > GMM_WS_TICKET) return 1;
  int best = 1, best_cost = nk * 16;                          // costs in sixteenths of a K tile
  for (int S = 2; S <= GMM_SPLIT_MAX; ++S) {
    if (S * tail > max_parts || nk / S < GMM_SPLIT_PART_MIN) break;
    const int turns = (tail * S + W - 1) / W;
    const int cost = turns * ((nk * 16 + S - 1) / S + GMM_SPLIT_PART_COST * 16);
    if (cost < best_cost) { best = S; best_cost = cost; }
  }
  return (best > 1 && best_cost * 5 <= nk * 16 * 4) ? best : 1;
}

// K tiles [first, last) of part `part` of S of a tile with nk K tiles.
GMM_HD void gmm_part_ktiles(int nk, int S, int part, int& first, int& last) {
  first = int(int64_t(part) * nk / S);
  last = int(int64_t(part + 1) * nk / S);
}

// [lo, hi) of group g along the jagged dimension, clamped into [0, extent] and
// made non-decreasing so that malformed offsets can never index out of bounds.
GMM_HD void gmm_group_range(const int32_t* offs, int g, int extent, int& lo, int& hi) {
  int s = g > 0 ? offs[g - 1] : 0;
  int e = offs[g];
  s = gmm_min(gmm_max(s, 0), extent);
  e = gmm_min(gmm_max(e, 0), extent);
  if (e < s) e = s;
  lo = s;
  hi = e;
}

// Tile grid of one group.  Along a jagged M or N the first tile starts at
// lo rounded down to `align`, so that vector loads stay aligned in memory.
GMM_HD void gmm_group_grid(int jag, int lo, int hi, int M, int N, int bm, int bn, int align,
                           int& tiles_m, int& tiles_n) {
  tiles_m = gmm_cdiv(M, bm);
  tiles_n = gmm_cdiv(N, bn);
  if (jag == GMM_JAG_M) tiles_m = hi > lo ? gmm_cdiv(hi - (lo / align) * align, bm) : 0;
  if (jag == GMM_JAG_N) tiles_n = hi > lo ? gmm_cdiv(hi - (lo / align) * align, bn) : 0;
}

// Upper bound on the number of tiles of a launch that needs no look at the offsets (the host uses it to
// launch fewer workgroups for small problems; a grid larger than the tile count only costs start-up
// time).  bm = smallest tile height in use.  Every group can add a partial tile at its end, one for the
// aligned-down start and one remainder tile: three per group on top of the even split.
GMM_HD int64_t gmm_tile_bound(int jag, int G, int M, int N, int bm, int bn) {
  const int64_t tm = gmm_cdiv(M, bm), tn = gmm_cdiv(N, bn);
  if (jag == GMM_JAG_M) return (int64_t(M) / bm + 3 * int64_t(G)) * tn;
  if (jag == GMM_JAG_N) return (int64_t(N) / bn + 3 * int64_t(G)) * (tm + 1);
  return int64_t(G) * (tm + 1) * tn;
}

// Linear id inside a group -> (tile row, tile column).  Tile rows advance
// fastest inside bands of GMM_BAND rows, so tiles that run at the same time
// share a few A row panels and a few B column panels.
GMM_HD void gmm_decode_in_group(int t, int tiles_m, int tiles_n, int& mt, int& nt) {
  const int per_band = GMM_BAND * tiles_n;
  const int band = t / per_band;
  const int first = band * GMM_BAND;
  const int rows = gmm_min(tiles_m - first, GMM_BAND);
  const int r = t - band * per_band;
  mt = first + r % rows;
  nt = r / rows;
}

// Renumbering for the 8 XCDs of the chip.  Workgroup w runs on XCD w % 8 and
// takes tiles w, w + num_wg, ...; inside every span of `num_wg` consecutive ids
// the ids handled by one XCD are made contiguous, so that each XCD's L2 sees a
// compact block of the tile grid.  `num_wg` must be a multiple of 8.  It is a
// permutation of [0, total).
GMM_HD int gmm_xcd_remap(int t, int total, int num_wg) {
  const int span = t / num_wg;
  const int base = span * num_wg;
  const int len = gmm_min(total - base, num_wg);
  const int r = t - base;
  const int x = r & 7;
  // ids of XCD y in this span: those r < len with r % 8 == y, i.e. (len - y + 7) / 8 of them
  const int q = len >> 3, rem = len & 7;
  const int start = x * q + gmm_min(x, rem);
  return base + start + (r >> 3);
}

// Group that holds linear tile id t, given the exclusive prefix sum cum[0..G]:
// the g with cum[g] <= t < cum[g + 1] (empty groups are skipped by construction).
GMM_HD int gmm_find_group(const int32_t* cum, int G, int t) {
  int lo = 0, hi = G;  // invariant: cum[lo] <= t < cum[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cum[mid] <= t) lo = mid; else hi = mid;
  }
  return lo;
}

// ---- tile heights ------------------------------------------------------------------------------ //
// Skewed group sizes leave many groups far smaller than a tall tile.  The row range of a group is cut
// into tall tiles; a remainder that fits one shorter tile (64 rows, or 128 under 256-row tall tiles)
// becomes one: it streams B at the same rate but wastes less MFMA work on rows that do not exist.  A
// shorter tile runs slower per row (measured: a 128-row tile costs about 0.76 of a 256-row one -- half the
// MFMAs for three quarters of the copies per K tile -- and a 64-row tile little less, both being bound by the
// stream of their B panel), so a remainder that needs two of them pays for another tall tile instead.
// All tall tiles of all groups come first in the tile order, the remainder tiles fill the tail of the
// launch (or, group_major, every group's remainder tile follows its tall tiles).
// `rem_rows` is the height of the group's remainder tile (n_short is 0 or 1).
GMM_HD void gmm_split_rows(int rows, int tall, int shrt, int& n_tall, int& n_short, int& rem_rows) {
  rem_rows = shrt;
  if (rows <= 0) { n_tall = 0; n_short = 0; return; }
  if (shrt <= 0) { n_tall = gmm_cdiv(rows, tall); n_short = 0; return; }
  n_tall = rows / tall;
  n_short = 0;
  const int rem = rows - n_tall * tall;
  if (rem == 0) return;
  if (rem <= shrt) { n_short = 1; }
  else if (tall > 2 * shrt && rem <= 2 * shrt) { n_short = 1; rem_rows = 2 * shrt; }
  else n_tall += 1;
}

// Rows of group g that the tile grid has to span (from the aligned-down start when rows are jagged).
GMM_HD int gmm_group_rows(int jag, int lo, int hi, int M, int align) {
  if (jag != GMM_JAG_M) return M;
  return hi > lo ? hi - (lo / align) * align : 0;
}

// Tile columns of group g (from the aligned-down start when columns are jagged).
GMM_HD int gmm_group_tile_cols(int jag, int lo, int hi, int N, int align, int bn) {
  if (jag != GMM_JAG_N) return gmm_cdiv(N, bn);
  return hi > lo ? gmm_cdiv(hi - (lo / align) * align, bn) : 0;
}

// One output tile, in global coordinates of the operands.
struct GmmTile {
  int32_t g;
  int32_t m0, n0;        // origin of the tile
  int32_t m_lo, m_hi;    // rows that may be stored: [m_lo, m_hi)
  int32_t n_lo, n_hi;    // columns that may be stored
  int32_t k_lo, k_hi;    // contraction range that contributes
  int32_t rows;          // height of the tile (0: the kernel's only height)
  int32_t part, nparts;    // part `part` of `nparts` along K (nparts 1: the whole tile); tail_idx: index of the tile
  int32_t tail_idx;        // in the split round (its arrival counter)
  int32_t share, sharers;  // the tile is number `share` of the `sharers` tiles of its band that read the same
                           // panel of the second operand at the same time (L2 prefetch shares); 0 sharers: none
};

GMM_HD GmmTile gmm_make_tile(const GmmParams& p, int g, int lo, int hi, int mt, int nt, int bm, int bn) {
  GmmTile t;
  t.g = g;
  t.rows = 0;
  t.share = 0; t.sharers = 0;
  t.part = 0; t.nparts = 1; t.tail_idx = 0;
  t.m0 = mt * bm; t.m_lo = 0; t.m_hi = p.M;
  t.n0 = nt * bn; t.n_lo = 0; t.n_hi = p.N;
  t.k_lo = 0; t.k_hi = p.K;
  if (p.jag == GMM_JAG_M) { t.m0 += (lo / p.align) * p.align; t.m_lo = lo; t.m_hi = hi; }
  if (p.jag == GMM_JAG_N) { t.n0 += (lo / p.align) * p.align; t.n_lo = lo; t.n_hi = hi; }
  if (p.jag == GMM_JAG_K) { t.k_lo = lo; t.k_hi = hi; }
  return t;
}

// Tile of the list above: `cls` 0 = tall, 1 = remainder tile; `local` = index inside the group's tiles of
// that class.
GMM_HD GmmTile gmm_make_tile2(const GmmParams& p, int g, int lo, int hi, int cls, int local, int bn) {
  const int rows = gmm_group_rows(p.jag, lo, hi, p.M, p.align);
  int n_tall, n_short, rem_rows;
  gmm_split_rows(rows, p.tall, p.shrt, n_tall, n_short, rem_rows);
  const int tn = gmm_group_tile_cols(p.jag, lo, hi, p.N, p.align, bn);
  int mt = 0, nt = local, m_off = n_tall * p.tall;
  if (cls == 0) {
    gmm_decode_in_group(local, n_tall, tn, mt, nt);
    m_off = mt * p.tall;
  }
  GmmTile t = gmm_make_tile(p, g, lo, hi, 0, nt, p.tall, bn);
  t.m0 += m_off;
  t.rows = cls == 0 ? p.tall : rem_rows;
  if (cls == 0) {
    const int first = (mt / GMM_BAND) * GMM_BAND;
    t.share = mt - first;
    t.sharers = gmm_min(n_tall - first, GMM_BAND);
  }
  return t;
}
