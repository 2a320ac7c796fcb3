// Persistent bf16 MFMA grouped GEMM for gfx950 (MI355X).
//
// One kernel body serves the four variants: the tile list (gmm_sched.h) turns a
// linear tile id into a group, an origin and the row / column / contraction
// ranges that the group owns, and the main loop is an ordinary C = A * B tile.
//
//   * v_mfma_f32_32x32x16_bf16, fp32 accumulators, one rounding at the end;
//   * A and B tiles are staged in LDS as [row][64 k] with 16-byte chunks
//     XOR-swizzled against bank conflicts, two buffers, one barrier per k-tile;
//   * an operand that is contiguous along K is copied chunk by chunk; one that
//     is contiguous along M or N (row-major B, column-major A) is read with
//     16-byte loads along its contiguous dimension and transposed 8 x 8 in
//     registers (v_perm) before it is written to LDS, so both layouts feed the
//     same MFMA fragment reads;
//   * stores are masked to the rows / columns the tile's own group owns, so no
//     second "fix-up" launch is needed (the reference needs one:
//     grouped_mm_bf16/kernels.py:363-419) and nothing outside a group is written.
//
// Requirements checked by the host before this family is chosen: bf16 inputs,
// 16-byte aligned bases, leading dimensions and contiguous extents that are
// multiples of 8 elements.
#include "gmm_device.h"
#include "gmm_launch.h"
#include "gmm_tile.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BK = 64;  // contraction elements per LDS tile (8 chunks of 16 bytes per row)

// Swizzle of the 16-byte chunk index inside a 128-byte LDS row.
__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }

__device__ __forceinline__ int lds_off(int row, int chunk) { return row * BK + ((chunk ^ swz(row)) << 3); }

__device__ __forceinline__ uint4 zero4() { return make_uint4(0, 0, 0, 0); }

// Keep elements e of a chunk with lo_e <= e < hi_e, zero the rest.
__device__ __forceinline__ uint4 mask_chunk(uint4 v, int lo_e, int hi_e) {
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t m0 = (2 * i >= lo_e && 2 * i < hi_e) ? 0x0000ffffu : 0u;
    const uint32_t m1 = (2 * i + 1 >= lo_e && 2 * i + 1 < hi_e) ? 0xffff0000u : 0u;
    w[i] &= (m0 | m1);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// ---- global -> register -> LDS staging of one ROWS x 64 operand tile ------ //

// Operand contiguous along K: element (row, k) at base[row * ld + k].
template <int ROWS, int NT>
struct StageKC {
  static constexpr int PER = (ROWS * 8 + NT - 1) / NT;
  uint4 r[PER];

  __device__ __forceinline__ void load(const uint16_t* base, int64_t ld, int row0, int row_ext, int kk,
                                       int k_lo, int k_hi, bool elem_mask) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int it = 0; it < PER; ++it) {
      const int q = it * NT + tid;
      const int row = q >> 3, c = q & 7;
      uint4 v = zero4();
      if (ROWS * 8 % NT == 0 || q < ROWS * 8) {
        const int rg = gmm_min(row0 + row, row_ext - 1);
        const int kc = kk + c * 8;
        if (kc < k_hi && kc + 8 > k_lo) {
          v = *reinterpret_cast<const uint4*>(base + int64_t(rg) * ld + kc);
          if (elem_mask) v = mask_chunk(v, k_lo - kc, k_hi - kc);
        }
      }
      r[it] = v;
    }
  }

  __device__ __forceinline__ void store(uint16_t* lds) const {
    const int tid = threadIdx.x;
#pragma unroll
    for (int it = 0; it < PER; ++it) {
      const int q = it * NT + tid;
      const int row = q >> 3, c = q & 7;
      if (ROWS * 8 % NT == 0 || q < ROWS * 8) *reinterpret_cast<uint4*>(lds + lds_off(row, c)) = r[it];
    }
  }
};

// Operand contiguous along its row index (M for A, N for B): element (row, k)
// at base[k * ld + row].  Each thread owns 8 rows x 8 k and transposes them.
template <int ROWS, int NT>
struct StageMC {
  static constexpr int BLOCKS = ROWS;  // (ROWS / 8) row blocks x 8 k blocks
  static constexpr int PER = (BLOCKS + NT - 1) / NT;
  uint4 r[PER][8];

  __device__ __forceinline__ void load(const uint16_t* base, int64_t ld, int row0, int row_ext, int kk,
                                       int k_lo, int k_hi, bool) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int it = 0; it < PER; ++it) {
      const int blk = it * NT + tid;
      const int rb = blk % (ROWS / 8), kb = blk / (ROWS / 8);
      int rg = row0 + rb * 8;
      if (rg + 8 > row_ext) rg = row_ext - 8;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = kk + kb * 8 + j;
        uint4 v = zero4();
        if ((BLOCKS % NT == 0 || blk < BLOCKS) && k >= k_lo && k < k_hi)
          v = *reinterpret_cast<const uint4*>(base + int64_t(k) * ld + rg);
        r[it][j] = v;
      }
    }
  }

  __device__ __forceinline__ void store(uint16_t* lds) const {
    const int tid = threadIdx.x;
#pragma unroll
    for (int it = 0; it < PER; ++it) {
      const int blk = it * NT + tid;
      const int rb = blk % (ROWS / 8), kb = blk / (ROWS / 8);
      if (!(BLOCKS % NT == 0 || blk < BLOCKS)) continue;
      const uint32_t* w = reinterpret_cast<const uint32_t*>(&r[it][0]);  // w[j * 4 + p]: k row j, word p
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        // output row i (operand row rb * 8 + i): 8 k values, two per word
        const int pw = i >> 1;
        const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
        uint4 o;
        o.x = __builtin_amdgcn_perm(w[1 * 4 + pw], w[0 * 4 + pw], sel);
        o.y = __builtin_amdgcn_perm(w[3 * 4 + pw], w[2 * 4 + pw], sel);
        o.z = __builtin_amdgcn_perm(w[5 * 4 + pw], w[4 * 4 + pw], sel);
        o.w = __builtin_amdgcn_perm(w[7 * 4 + pw], w[6 * 4 + pw], sel);
        *reinterpret_cast<uint4*>(lds + lds_off(rb * 8 + i, kb)) = o;
      }
    }
  }
};

template <bool KC, int ROWS, int NT> struct StageSel { typedef StageKC<ROWS, NT> type; };
template <int ROWS, int NT> struct StageSel<false, ROWS, NT> { typedef StageMC<ROWS, NT> type; };

__device__ __forceinline__ void store_out(float* c, int64_t idx, float v) { c[idx] = v; }
__device__ __forceinline__ void store_out(uint16_t* c, int64_t idx, float v) { c[idx] = gmm_bf16_bits(v); }

template <int BM, int BN, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC, typename OutT>
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64, 1) gmm_mfma_kernel(const GmmParams p) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of the MFMA tile");

  __shared__ __attribute__((aligned(16))) uint16_t lds_a[2][BM * BK];
  __shared__ __attribute__((aligned(16))) uint16_t lds_b[2][BN * BK];
  __shared__ int32_t cum[GMM_MAX_GROUPS + 1];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;

  const int total = gmm_build_tile_table<NT>(p, BM, BN, cum);
  const uint16_t* __restrict__ A = static_cast<const uint16_t*>(p.a);
  const uint16_t* __restrict__ B = static_cast<const uint16_t*>(p.b);
  OutT* __restrict__ C = static_cast<OutT*>(p.c);
  const int64_t a_ld = A_KC ? p.a_sm : p.a_sk;
  const int64_t b_ld = B_KC ? p.b_sn : p.b_sk;

  typename StageSel<A_KC, BM, NT>::type sa;
  typename StageSel<B_KC, BN, NT>::type sb;

  for (int t = blockIdx.x; t < total; t += gridDim.x) {
    const int tt = p.xcd_remap ? gmm_xcd_remap(t, total, gridDim.x) : t;
    const GmmTile tile = gmm_locate_tile(p, cum, tt, BM, BN);
    const uint16_t* a = A + int64_t(tile.g) * p.a_sg;
    const uint16_t* b = B + int64_t(tile.g) * p.b_sg;
    OutT* c = C + int64_t(tile.g) * p.c_sg;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    const int k_begin = tile.k_lo & ~7;
    const int nk = tile.k_hi > tile.k_lo ? gmm_cdiv(tile.k_hi - k_begin, BK) : 0;
    const bool elem_mask = ((tile.k_lo | tile.k_hi) & 7) != 0;

    if (nk > 0) {
      sa.load(a, a_ld, tile.m0, p.M, k_begin, tile.k_lo, tile.k_hi, elem_mask);
      sb.load(b, b_ld, tile.n0, p.N, k_begin, tile.k_lo, tile.k_hi, elem_mask);
      sa.store(lds_a[0]);
      sb.store(lds_b[0]);
      __syncthreads();
    }
    for (int kt = 0; kt < nk; ++kt) {
      const int cur = kt & 1;
      const bool more = kt + 1 < nk;
      if (more) {
        const int kk = k_begin + (kt + 1) * BK;
        sa.load(a, a_ld, tile.m0, p.M, kk, tile.k_lo, tile.k_hi, elem_mask);
        sb.load(b, b_ld, tile.n0, p.N, kk, tile.k_lo, tile.k_hi, elem_mask);
      }
      const uint16_t* la = lds_a[cur];
      const uint16_t* lb = lds_b[cur];
#pragma unroll
      for (int s = 0; s < BK / 16; ++s) {
        bf16x8 af[TM], bf[TN];
        const int chunk = 2 * s + (lane >> 5);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const int row = wm * WTM + i * 32 + (lane & 31);
          af[i] = *reinterpret_cast<const bf16x8*>(la + lds_off(row, chunk));
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int row = wn * WTN + j * 32 + (lane & 31);
          bf[j] = *reinterpret_cast<const bf16x8*>(lb + lds_off(row, chunk));
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
      }
      if (more) {
        sa.store(lds_a[cur ^ 1]);
        sb.store(lds_b[cur ^ 1]);
      }
      __syncthreads();
    }

    // Epilogue: lane holds, for each 32 x 32 block, column (lane % 32) and rows
    // 8 q + 4 (lane / 32) + r for q, r in 0..3.
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = tile.m0 + wm * WTM + i * 32 + 8 * q + 4 * (lane >> 5) + r;
          const bool row_ok = row >= tile.m_lo && row < tile.m_hi;
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            const int col = tile.n0 + wn * WTN + j * 32 + (lane & 31);
            if (row_ok && col >= tile.n_lo && col < tile.n_hi)
              store_out(c, int64_t(row) * p.c_sm + int64_t(col) * p.c_sn, acc[i][j][4 * q + r]);
          }
        }
      }
    }
  }
}


// 16 bytes read at device scope (sc1): served by memory or the Infinity Cache, never by a stale line of this
// XCD's L2.  Buffer loads, so that the compiler pipelines them and tracks their completion itself.
typedef unsigned gmm_u4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 gmm_load_device_scope(__amdgpu_buffer_rsrc_t rsrc, unsigned byte_offset) {
  const gmm_u4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, int(byte_offset), 0, 16 /* sc1 */);
  return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}

// ---- last part of a split tile: add the partial tiles and store the output ------------------------ //
// The parts of a tile (gmm_tail_split) leave fp32 partial tiles of `rows` x 256 in the workspace, part j of
// tile number `tail_idx` of the split round in slot j * tail + tail_idx.  Every part, once its partial is
// visible to the whole device, counts itself on the tile's arrival counter; the one that finds all others
// there adds the partials in part order (so the sum is the same whichever part comes last), rounds once and
// stores the rows and columns the tile's group owns.  It leaves the counter at zero for the next launch.
// Nobody waits for anybody.  All threads of the workgroup must call it.
template <int OUT_F32, int F16>
__device__ __forceinline__ void gmm_split_finish(const GmmParams& p, char* c_group, int ldc, int m0, int n0, int m_lo,
                                                 int m_hi, int n_lo, int n_hi, int rows, int nparts, int tail,
                                                 int tail_idx, int* flag) {
  const int tid = threadIdx.x;
  unsigned* counters = static_cast<unsigned*>(p.ws);
  // the slots of this tile's parts, addressed from slot `tail_idx` (parts are `tail` slots apart)
  const __amdgpu_buffer_rsrc_t slots = __builtin_amdgcn_make_buffer_rsrc(
      static_cast<char*>(p.ws) + GMM_WS_HEADER + size_t(tail_idx) * GMM_WS_SLOT, 0, 0x7fffffff, 0x00020000);
  // The partial tile was stored through to memory at device scope; once this thread's stores are done they
  // are visible to every workgroup that reads at device scope (no L2 has to be written back or invalidated).
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (tid == 0)
    *flag = int(__hip_atomic_fetch_add(&counters[tail_idx], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  __syncthreads();
  const bool last = *flag == nparts - 1;
  __syncthreads();   // everybody has read the flag before a later tile overwrites it
  if (!last) return;
  if (tid == 0) __hip_atomic_store(&counters[tail_idx], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const int r_end = gmm_min(m_hi, m0 + rows) - m0;       // rows of the tile at or past it belong to nobody here
  const int r_begin = gmm_max(m_lo - m0, 0);
  const int chunk = tid & 63;                             // 4 columns: 4 chunk .. 4 chunk + 3
  const int col = n0 + 4 * chunk;
  int valid = 0;
#pragma unroll
  for (int e = 0; e < 4; ++e) valid |= (col + e >= n_lo && col + e < n_hi) ? (1 << e) : 0;
  if (valid == 0) return;
  // Four rows per thread at a time: their 4 * nparts loads are in flight together (each is a trip to the
  // Infinity Cache or to memory; one row at a time, the loop is 64 such trips long).
  constexpr int ROWS_AT_ONCE = 4;
  for (int r0 = r_begin + (tid >> 6); r0 < r_end; r0 += 4 * ROWS_AT_ONCE) {
    float4 part[ROWS_AT_ONCE][GMM_SPLIT_MAX];
#pragma unroll
    for (int u = 0; u < ROWS_AT_ONCE; ++u) {
      const int r = r0 + 4 * u;
      const unsigned at_slot = unsigned(r * 256 + 4 * chunk) * 4;
#pragma unroll
      for (int j = 0; j < GMM_SPLIT_MAX; ++j)
        if (j < nparts && r < r_end) part[u][j] = gmm_load_device_scope(slots, unsigned(j * tail) * unsigned(GMM_WS_SLOT) + at_slot);
    }
#pragma unroll
    for (int u = 0; u < ROWS_AT_ONCE; ++u) {
      const int r = r0 + 4 * u;
      if (r >= r_end) break;
      float4 acc = part[u][0];
#pragma unroll
      for (int j = 1; j < GMM_SPLIT_MAX; ++j)
        if (j < nparts) { acc.x += part[u][j].x; acc.y += part[u][j].y; acc.z += part[u][j].z; acc.w += part[u][j].w; }
      const float f[4] = {acc.x, acc.y, acc.z, acc.w};
      const size_t at = size_t(m0 + r) * ldc + col;
      if constexpr (OUT_F32) {
        float* out = reinterpret_cast<float*>(c_group) + at;
        if (valid == 15) *reinterpret_cast<float4*>(out) = acc;
        else
#pragma unroll
          for (int e = 0; e < 4; ++e) if (valid & (1 << e)) out[e] = f[e];
      } else {
        uint16_t h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if constexpr (F16) { const _Float16 x = _Float16(f[e]); h[e] = *reinterpret_cast<const uint16_t*>(&x); }
          else h[e] = gmm_bf16_bits(f[e]);
        }
        uint16_t* out = reinterpret_cast<uint16_t*>(c_group) + at;
        if (valid == 15) *reinterpret_cast<uint2*>(out) = make_uint2(h[0] | (uint32_t(h[1]) << 16), h[2] | (uint32_t(h[3]) << 16));
        else
#pragma unroll
          for (int e = 0; e < 4; ++e) if (valid & (1 << e)) out[e] = h[e];
      }
    }
  }
}

// ---- kernel built on the generated assembly tile (gmm_tile.h) --------------------------------- //
// Same tile list, but each tile's main loop and epilogue run as one hand-scheduled assembly block:
// direct global -> LDS copies, no register staging, explicit registers.  A_TR / B_TR: the operand is
// contiguous along M / N (not along K) and is read from LDS with transposing loads.
// One wave per SIMD; tiles of 256, 128 and 64 rows share the launch when A is contiguous along K (a
// column-major A has only the first): p.tall is the height of the tall tiles (256 or 128), p.shrt == 64
// turns on the 64-row tiles for group remainders.
// A located tile as the workgroup keeps it in LDS between locating and running it.
struct GmmTileRec {
  int32_t g, m0, n0, m_lo, m_hi, n_lo, n_hi, k_lo, k_hi, rows;
  int32_t shares;   // share | sharers << 8 (L2 prefetch of B)
  int32_t part;     // part | tail_idx << 8 for a part of a tile cut along K, else -1
};

__device__ __forceinline__ void gmm_store_rec(GmmTileRec* d, const GmmTile& tile, int part) {
  d->g = tile.g; d->m0 = tile.m0; d->n0 = tile.n0; d->m_lo = tile.m_lo; d->m_hi = tile.m_hi;
  d->n_lo = tile.n_lo; d->n_hi = tile.n_hi; d->k_lo = tile.k_lo; d->k_hi = tile.k_hi; d->rows = tile.rows;
  d->shares = tile.share | (tile.sharers << 8);
  d->part = part;
}

// The record read back as scalars (every lane reads the same words).
struct GmmTileScalars {
  int g, m0, n0, m_lo, m_hi, n_lo, n_hi, k_lo, k_hi, rows, shares, part;
};

__device__ __forceinline__ GmmTileScalars gmm_load_rec(const GmmTileRec* d) {
  GmmTileScalars t;
  t.g = __builtin_amdgcn_readfirstlane(d->g);
  t.m0 = __builtin_amdgcn_readfirstlane(d->m0); t.n0 = __builtin_amdgcn_readfirstlane(d->n0);
  t.m_lo = __builtin_amdgcn_readfirstlane(d->m_lo); t.m_hi = __builtin_amdgcn_readfirstlane(d->m_hi);
  t.n_lo = __builtin_amdgcn_readfirstlane(d->n_lo); t.n_hi = __builtin_amdgcn_readfirstlane(d->n_hi);
  t.k_lo = __builtin_amdgcn_readfirstlane(d->k_lo); t.k_hi = __builtin_amdgcn_readfirstlane(d->k_hi);
  t.rows = __builtin_amdgcn_readfirstlane(d->rows);
  t.shares = __builtin_amdgcn_readfirstlane(d->shares);
  t.part = __builtin_amdgcn_readfirstlane(d->part);
  return t;
}

// Operands of a tile for the assembly.  CDIV = 2 for the SwiGLU epilogue (256 columns of the product become
// 128 columns of the output), ESZ = bytes per output element.
template <int A_TR, int B_TR, int ESZ, int CDIV>
__device__ __forceinline__ GmmTileDesc gmm_describe_tile(const GmmParams& p, const GmmTileScalars& t) {
  const int lda = int(A_TR ? p.a_sk : p.a_sm);
  const int ldb = int(B_TR ? p.b_sk : p.b_sn);
  const int ldc = int(p.c_sm);
  // the copies move 16-byte chunks along K for an operand that is contiguous along K
  const int k_begin = (A_TR && B_TR) ? t.k_lo : (t.k_lo & ~7);
  const uint16_t* a = static_cast<const uint16_t*>(p.a) + int64_t(t.g) * p.a_sg;
  const uint16_t* b = static_cast<const uint16_t*>(p.b) + int64_t(t.g) * p.b_sg;
  GmmTileDesc dsc;
  dsc.a.ld = lda;
  dsc.b.ld = ldb;
  // Extents end at the last element of the operand's last row, not at a whole leading dimension: a
  // padded view (ld larger than the row) may end exactly there.
  if (!A_TR && p.gather) {
    // row gather: the tile's rows come from rows gather[m0 ..] of the whole source matrix
    dsc.a.base = a + k_begin;
    dsc.a.bytes = (int64_t(p.a_rows - 1) * lda + (p.K - k_begin)) * 2;
    dsc.a.gather = p.gather + t.m0;
    dsc.a.gather_n = t.m_hi - t.m0;
    dsc.a.src_rows = p.a_rows;
  } else if (!A_TR) {
    // rows past the group's last row (jagged rows) are not fetched at all: they read as zeros
    const int a_rows_end = p.jag == GMM_JAG_M ? t.m_hi : p.M;
    dsc.a.base = a + int64_t(t.m0) * lda + k_begin;
    dsc.a.bytes = (int64_t(a_rows_end - 1 - t.m0) * lda + (p.K - k_begin)) * 2;
  } else {
    dsc.a.base = a + int64_t(k_begin) * lda + t.m0;
    dsc.a.bytes = (int64_t(p.K - 1 - k_begin) * lda + (p.M - t.m0)) * 2;
  }
  if (!B_TR) {
    dsc.b.base = b + int64_t(t.n0) * ldb + k_begin;
    dsc.b.bytes = (int64_t(p.N - 1 - t.n0) * ldb + (p.K - k_begin)) * 2;
  } else {
    dsc.b.base = b + int64_t(k_begin) * ldb + t.n0;
    dsc.b.bytes = (int64_t(p.K - 1 - k_begin) * ldb + (p.N - t.n0)) * 2;
  }
  dsc.c = static_cast<char*>(p.c) + (int64_t(t.g) * p.c_sg + int64_t(t.m0) * ldc + t.n0 / CDIV) * ESZ;
  dsc.ldc = ldc;
  dsc.c_bytes = (int64_t(p.M - 1 - t.m0) * ldc + (p.N - t.n0) / CDIV) * ESZ;
  dsc.klen = t.k_hi > t.k_lo ? t.k_hi - k_begin : 0;
  dsc.khead = t.k_lo - k_begin;
  dsc.row_rel0 = t.m0 - t.m_lo;
  // rows past the tile's own height belong to the next tile of the group
  dsc.row_cnt = gmm_min(t.m_hi, t.m0 + t.rows) - t.m_lo;
  dsc.col_lo = gmm_max(t.n_lo - t.n0, 0) / CDIV;
  dsc.col_hi = gmm_min(t.n_hi - t.n0, GMM_TILE_N) / CDIV;
  dsc.share = t.shares & 0xff;
  dsc.sharers = t.shares >> 8;
  return dsc;
}

template <int A_TR, int B_TR, int OUT_F32, int F16, int ACT = 0>
__global__ void __launch_bounds__(256, 1) gmm_asm_kernel(const GmmParams p) {
  constexpr int WAVES = 4;
  constexpr bool SHORT_TILES = !A_TR;
  constexpr int LDS_256 = gmm_tile_lds_bytes<A_TR, B_TR, 4>();
  constexpr int LDS_128 = SHORT_TILES ? gmm_tile_lds_bytes<0, B_TR, 2>() : 0;
  constexpr int LDS_64 = SHORT_TILES ? gmm_tile_lds_bytes<0, B_TR, 1>() : 0;
  constexpr int LDS_MAX = LDS_256 > LDS_128 ? (LDS_256 > LDS_64 ? LDS_256 : LDS_64) : (LDS_128 > LDS_64 ? LDS_128 : LDS_64);
  constexpr int BATCH = 32;  // tiles located at a time
  __shared__ __attribute__((aligned(1024))) char lds[LDS_MAX];
  __shared__ int32_t cum_tall[GMM_MAX_GROUPS + 1];
  __shared__ int32_t cum_short[GMM_MAX_GROUPS + 1];
  __shared__ GmmTileRec tiles[BATCH];
  __shared__ int32_t split_flag;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) char*)lds;
  constexpr int ESZ = OUT_F32 ? 4 : 2;
  constexpr int CDIV = ACT ? 2 : 1;

  int total_tall;
  const int total_tiles = gmm_build_tile_table2<WAVES * 64>(p, GMM_TILE_N, cum_tall, cum_short, total_tall);
  // The tiles of the last, partly filled round may be cut along K into `nparts` parts each (gmm_tail_split).
  // Tiles before split_base are dealt round-robin (workgroup w takes w, w + grid, ...); the parts are taken
  // from a ticket counter in the workspace by whichever workgroup is free: part q is K part q / tail of tile
  // split_base + q % tail.
  int nparts = 1, tail = 0;
  if (!ACT && p.ws_parts > 0 && p.jag != GMM_JAG_K) {
    nparts = gmm_tail_split(total_tiles, int(gridDim.x), gmm_cdiv(p.K, GMM_TILE_K), p.ws_parts);
    if (nparts > 1) tail = total_tiles % int(gridDim.x);
  }
  const int split_base = total_tiles - tail;       // == total_tiles when nothing is cut

  // Locating a tile (binary search over the groups, reads of offs, integer divisions) costs microseconds, so
  // BATCH threads locate the next BATCH round-robin tiles of the workgroup at once and leave them in LDS for
  // the tile loop to pick up.
  for (int first = 0;; first += BATCH) {
    const int64_t mine = int64_t(blockIdx.x) + int64_t(first + tid) * gridDim.x;
    if (tid < BATCH && mine < split_base) {
      const int t = int(mine);
      const int tt = p.xcd_remap ? gmm_xcd_remap(t, split_base, gridDim.x) : t;
      gmm_store_rec(&tiles[tid], gmm_locate_tile2(p, cum_tall, cum_short, total_tall, tt, GMM_TILE_N), -1);
    }
    __syncthreads();
    const int64_t left = (int64_t(split_base) - blockIdx.x + gridDim.x - 1) / gridDim.x - first;  // tiles of this workgroup from `first` on
    const int here = left < BATCH ? int(left) : BATCH;
    for (int j = 0; j < here; ++j) {
      // Everything the assembly wants per lane is a cheap function of the lane id.  Hidden from the
      // optimiser per tile, or it hoists those values out of the loop, keeps them alive across the
      // assembly (which clobbers most registers) and spills them to scratch memory.
      int lane_j = lane;
      asm volatile("" : "+v"(lane_j));
      const GmmTileScalars t = gmm_load_rec(&tiles[j]);
      const GmmTileDesc dsc = gmm_describe_tile<A_TR, B_TR, ESZ, CDIV>(p, t);
      if constexpr (A_TR) {
        gmm_tile_compute<A_TR, B_TR, OUT_F32, 4, F16>(dsc, lds_base, lane_j, wave);
      } else {
        // a short tile that holds all rows of its group is the only reader of its B panel
        const bool sole = t.m_hi - t.m_lo <= t.rows;
        if (t.rows == 256) gmm_tile_compute<A_TR, B_TR, OUT_F32, 4, F16, 0, ACT>(dsc, lds_base, lane_j, wave);
        else if (t.rows == 128 && !sole) gmm_tile_compute<A_TR, B_TR, OUT_F32, 2, F16, 0, ACT>(dsc, lds_base, lane_j, wave);
        else if (t.rows == 128) gmm_tile_compute<A_TR, B_TR, OUT_F32, 2, F16, 1, ACT>(dsc, lds_base, lane_j, wave);
        else if (!sole) gmm_tile_compute<A_TR, B_TR, OUT_F32, 1, F16, 0, ACT>(dsc, lds_base, lane_j, wave);
        else gmm_tile_compute<A_TR, B_TR, OUT_F32, 1, F16, 1, ACT>(dsc, lds_base, lane_j, wave);
      }
    }
    if (left <= BATCH) break;
    __syncthreads();  // everyone is done with this batch of located tiles
  }

  // The parts of the tiles that were cut: drawn from the ticket counter, one at a time, located by the thread
  // that draws.  Each part's whole fp32 tile goes to its workspace slot; gmm_split_finish does the rest.
  if constexpr (!ACT) {
    if (nparts > 1) {
      unsigned* const ws_header = static_cast<unsigned*>(p.ws);
      const int n_parts = tail * nparts;
      for (;;) {
        __syncthreads();  // the previous record and flag are no longer in use
        if (tid == 0) {
          const unsigned q = __hip_atomic_fetch_add(&ws_header[GMM_WS_TICKET], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          split_flag = q < unsigned(n_parts) ? 1 : 0;
          if (q < unsigned(n_parts)) {
            const int part = int(q) / tail, tail_idx = int(q) - part * tail;
            GmmTile tile = gmm_locate_tile2(p, cum_tall, cum_short, total_tall, split_base + tail_idx, GMM_TILE_N);
            int kt0, kt1;
            gmm_part_ktiles(gmm_cdiv(p.K, GMM_TILE_K), nparts, part, kt0, kt1);
            tile.k_lo = kt0 * GMM_TILE_K;
            tile.k_hi = gmm_min(kt1 * GMM_TILE_K, p.K);
            tile.sharers = 0;   // parts run out of step with their band: no prefetch shares
            gmm_store_rec(&tiles[0], tile, part | (tail_idx << 8));
          }
        }
        __syncthreads();
        if (!split_flag) break;
        int lane_j = lane;
        asm volatile("" : "+v"(lane_j));
        const GmmTileScalars t = gmm_load_rec(&tiles[0]);
        GmmTileDesc dsc = gmm_describe_tile<A_TR, B_TR, ESZ, 1>(p, t);
        const int tail_idx = t.part >> 8;
        dsc.c = static_cast<char*>(p.ws) + GMM_WS_HEADER + size_t((t.part & 0xff) * tail + tail_idx) * GMM_WS_SLOT;
        dsc.ldc = 256;
        dsc.c_bytes = GMM_WS_SLOT;
        dsc.row_rel0 = 0;
        dsc.row_cnt = t.rows;
        dsc.col_lo = 0;
        dsc.col_hi = GMM_TILE_N;
        if (A_TR || t.rows == 256) gmm_tile_compute<A_TR, B_TR, 1, 4, F16, 0, 2>(dsc, lds_base, lane_j, wave);
        else if (t.rows == 128) gmm_tile_compute<A_TR, B_TR, 1, A_TR ? 4 : 2, F16, 0, 2>(dsc, lds_base, lane_j, wave);
        else gmm_tile_compute<A_TR, B_TR, 1, A_TR ? 4 : 1, F16, 0, 2>(dsc, lds_base, lane_j, wave);
        gmm_split_finish<OUT_F32, F16>(p, static_cast<char*>(p.c) + int64_t(t.g) * p.c_sg * ESZ, int(p.c_sm), t.m0, t.n0,
                                       t.m_lo, t.m_hi, t.n_lo, t.n_hi, t.rows, nparts, tail, tail_idx, &split_flag);
      }
      // Every workgroup leaves the loop through exactly one ticket beyond the parts; the last one to leave
      // puts the ticket counter back to zero for the next launch.
      if (tid == 0) {
        const unsigned gone = __hip_atomic_fetch_add(&ws_header[GMM_WS_EXITED], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (gone == gridDim.x - 1) {
          __hip_atomic_store(&ws_header[GMM_WS_TICKET], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(&ws_header[GMM_WS_EXITED], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
  }
}

template <int OUT_F32, int F16>
int launch_asm(const GmmParams& p, GmmLayout lay, hipStream_t stream) {
  const dim3 grid(p.num_wg), block(256);
  if (p.act) {
    if constexpr (OUT_F32) {
      return -1;
    } else {
      if (!lay.a_kc) return -1;
      if (lay.b_kc)
        hipLaunchKernelGGL((gmm_asm_kernel<0, 0, 0, F16, 1>), grid, block, 0, stream, p);
      else
        hipLaunchKernelGGL((gmm_asm_kernel<0, 1, 0, F16, 1>), grid, block, 0, stream, p);
      return hipGetLastError() == hipSuccess ? 0 : 1;
    }
  }
  if (lay.a_kc && lay.b_kc)
    hipLaunchKernelGGL((gmm_asm_kernel<0, 0, OUT_F32, F16>), grid, block, 0, stream, p);
  else if (lay.a_kc && !lay.b_kc)
    hipLaunchKernelGGL((gmm_asm_kernel<0, 1, OUT_F32, F16>), grid, block, 0, stream, p);
  else if (!lay.a_kc && lay.b_kc)
    hipLaunchKernelGGL((gmm_asm_kernel<1, 0, OUT_F32, F16>), grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL((gmm_asm_kernel<1, 1, OUT_F32, F16>), grid, block, 0, stream, p);
  return hipGetLastError() == hipSuccess ? 0 : 1;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, typename OutT>
int launch_layout(const GmmParams& p, GmmLayout lay, hipStream_t stream) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  const dim3 grid(p.num_wg), block(NT);
  if (lay.a_kc && lay.b_kc)
    hipLaunchKernelGGL((gmm_mfma_kernel<BM, BN, WAVES_M, WAVES_N, true, true, OutT>), grid, block, 0, stream, p);
  else if (lay.a_kc && !lay.b_kc)
    hipLaunchKernelGGL((gmm_mfma_kernel<BM, BN, WAVES_M, WAVES_N, true, false, OutT>), grid, block, 0, stream, p);
  else if (!lay.a_kc && lay.b_kc)
    hipLaunchKernelGGL((gmm_mfma_kernel<BM, BN, WAVES_M, WAVES_N, false, true, OutT>), grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL((gmm_mfma_kernel<BM, BN, WAVES_M, WAVES_N, false, false, OutT>), grid, block, 0, stream, p);
  return hipGetLastError() == hipSuccess ? 0 : 1;
}

}  // namespace

int gmm_launch_mfma(GmmParams p, GmmLayout lay, int in_dtype, int out_dtype, int config, int num_cus, hipStream_t stream) {
  // persistent grid: one workgroup per CU, fewer (a multiple of 8, for the XCD renumbering) when the launch
  // cannot have that many tiles
  {
    const int64_t bound = gmm_tile_bound(p.jag, p.G, p.M, p.N, config == GMM_CFG_ASM_256x256 ? p.tall : 256, 256);
    const int64_t want = ((bound + 7) / 8) * 8;
    p.num_wg = int(want < num_cus ? (want < 8 ? 8 : want) : num_cus);
    // the tiles of a partly filled last round can be cut along K (gmm_tail_split); a launch of few tiles with a
    // long contraction gets the whole chip for that
    const bool can_split = config == GMM_CFG_ASM_256x256 && p.ws_parts > 0 && !p.act && p.jag != GMM_JAG_K &&
                           p.K >= 2 * GMM_SPLIT_PART_MIN * GMM_TILE_K;
    if (can_split && p.K >= 96 * GMM_TILE_K) p.num_wg = num_cus;
    if (!can_split) p.ws_parts = 0;
  }
  const bool out16 = out_dtype == in_dtype;   // else fp32
  if (!out16 && out_dtype != GMM_DT_F32) return -1;
  if (config == GMM_CFG_ASM_256x256) {
    // a column-major A has only the 256-row tile
    if (!lay.a_kc) { p.tall = 256; p.shrt = 0; }
    if (p.tall != 128) p.tall = 256;
    if (in_dtype == GMM_DT_BF16) return out16 ? launch_asm<0, 0>(p, lay, stream) : launch_asm<1, 0>(p, lay, stream);
    if (in_dtype == GMM_DT_F16) return out16 ? launch_asm<0, 1>(p, lay, stream) : launch_asm<1, 1>(p, lay, stream);
    return -1;
  }
  if (in_dtype != GMM_DT_BF16) return -1;     // the register-staged kernel is bf16 only
  if (out16) return launch_layout<256, 256, 2, 2, uint16_t>(p, lay, stream);
  return launch_layout<256, 256, 2, 2, float>(p, lay, stream);
}
