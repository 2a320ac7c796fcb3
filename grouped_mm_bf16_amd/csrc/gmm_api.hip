// C ABI of libgrouped_mm_hip.so (declared in include/grouped_mm_hip.h): argument
// checks, choice of kernel family, launch.  No allocation, no synchronisation,
// no exceptions across the boundary.
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "gmm_launch.h"

namespace {

std::atomic<int> g_forced_path{GMM_PATH_AUTO};
std::atomic<int> g_forced_config{-1};
std::atomic<int> g_xcd_remap{1};
std::atomic<int> g_forced_tall{-1};   // -1 auto, else 256 / 128
std::atomic<int> g_forced_short{-1};  // -1 auto, 0 off, 64 on
std::atomic<int> g_group_major{-1};   // -1 auto, 0 tall tiles of all groups first, 1 group by group
std::atomic<int> g_tail_split{1};     // 0: ignore the workspace (no tile is cut along K)
thread_local int t_last_path = 0;
thread_local int t_last_config = -1;

constexpr int kMaxDevices = 64;
std::atomic<int> g_num_cus[kMaxDevices];

int device_cus() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  int n = g_num_cus[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    n = (n / 8) * 8;  // the XCD renumbering wants a multiple of 8
    if (n <= 0) n = 8;
    g_num_cus[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

bool fits_i32(int64_t v) { return v >= 0 && v < (int64_t(1) << 31); }
bool mult8(int64_t v) { return (v & 7) == 0; }
bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

struct Problem {
  GmmParams p;
  int in_dtype, out_dtype;
};

// Caller's workspace -> split parameters: the header must fit, the slots must be 16-byte aligned.
void set_workspace(GmmParams& p, void* ws, int64_t bytes) {
  p.ws = nullptr;
  p.ws_parts = 0;
  if (!g_tail_split.load(std::memory_order_relaxed)) return;
  if (!ws || !aligned16(ws) || bytes < GMM_WS_HEADER + 2 * int64_t(GMM_WS_SLOT)) return;
  const int64_t parts = (bytes - GMM_WS_HEADER) / GMM_WS_SLOT;
  p.ws = ws;
  p.ws_parts = int32_t(parts > 4096 ? 4096 : parts);   // 32-bit byte offsets from a tile's first slot
}

// Decide whether the MFMA family can take the call, and with which operand layouts.
bool mfma_eligible(const Problem& pr, GmmLayout& lay, int& align) {
  const GmmParams& p = pr.p;
  if (pr.in_dtype != GMM_DT_BF16 && pr.in_dtype != GMM_DT_F16) return false;
  if (pr.out_dtype != pr.in_dtype && pr.out_dtype != GMM_DT_F32) return false;
  if (!aligned16(p.a) || !aligned16(p.b)) return false;
  if (!mult8(p.a_sg) || !mult8(p.b_sg)) return false;
  // A: contiguous along K (row-major) or along M (column-major)
  if (p.a_sk == 1 && mult8(p.a_sm) && mult8(p.K)) lay.a_kc = true;
  else if (p.a_sm == 1 && mult8(p.a_sk) && mult8(p.M) && p.M >= 8) lay.a_kc = false;
  else return false;
  // B: contiguous along K (column-major) or along N (row-major)
  if (p.b_sk == 1 && mult8(p.b_sn) && mult8(p.K)) lay.b_kc = true;
  else if (p.b_sn == 1 && mult8(p.b_sk) && mult8(p.N) && p.N >= 8) lay.b_kc = false;
  else return false;
  align = 1;
  if (p.jag == GMM_JAG_M && !lay.a_kc) align = 8;
  if (p.jag == GMM_JAG_N && !lay.b_kc) align = 8;
  return true;
}

// The generated-assembly tile takes a subset of what the register-staged kernel takes.
bool asm_tile_eligible(const Problem& pr, const GmmLayout& lay) {
  const GmmParams& p = pr.p;
  if (p.c_sn != 1) return false;
  const int64_t lda = lay.a_kc ? p.a_sm : p.a_sk, ldb = lay.b_kc ? p.b_sn : p.b_sk, ldc = p.c_sm;
  const int64_t ld_max = int64_t(1) << 22;
  if (lda >= ld_max || ldb >= ld_max || ldc >= ld_max) return false;
  // a transposed-layout operand is addressed from its first k row: the whole slice must fit 31 bits
  if (!lay.a_kc && int64_t(p.K) * lda * 2 >= (int64_t(1) << 31)) return false;
  if (!lay.b_kc && int64_t(p.K) * ldb * 2 >= (int64_t(1) << 31)) return false;
  // the epilogue stores 16-byte chunks of a row
  if (!aligned16(p.c)) return false;
  if (pr.out_dtype != GMM_DT_F32) {
    if (!mult8(p.c_sm) || !mult8(p.c_sg) || !mult8(p.N)) return false;
  } else {
    if ((p.c_sm & 3) || (p.c_sg & 3)) return false;
    if (ldc >= ld_max / 2) return false;   // 255 rows of 4-byte elements must stay below 2^31 bytes from the tile's origin
  }
  return true;
}

int run(Problem& pr, hipStream_t stream) {
  GmmParams& p = pr.p;
  if (p.G < 0 || (p.G >= GMM_MAX_GROUPS && p.jag != GMM_JAG_NONE)) return GMM_ERR_BAD_ARGUMENT;
  if (pr.in_dtype < 0 || pr.in_dtype > GMM_DT_F32) return GMM_ERR_UNSUPPORTED;
  if (pr.out_dtype != pr.in_dtype && pr.out_dtype != GMM_DT_F32) return GMM_ERR_UNSUPPORTED;
  // Nothing to write: no groups (the reference launches and stores nothing, kernels.py:162-172 with
  // G == 0 finds no owner for any row), or an empty extent.  Empty tensors may come with null pointers.
  if (p.G == 0 || p.M == 0 || p.N == 0) return GMM_OK;
  if (!p.a || !p.b || !p.c) return GMM_ERR_BAD_ARGUMENT;
  if (p.jag != GMM_JAG_NONE && !p.offs) return GMM_ERR_BAD_ARGUMENT;

  const int cus = device_cus();
  if (cus <= 0) return GMM_ERR_LAUNCH;

  GmmLayout lay{};
  int align = 1;
  const int forced = g_forced_path.load(std::memory_order_relaxed);
  const bool aligned = mfma_eligible(pr, lay, align);
  bool can_asm = aligned && asm_tile_eligible(pr, lay);
  // the SwiGLU epilogue exists on the assembly tile only: K-contiguous first operand, 16-bit output, whole
  // blocks of 64 gates + 64 partners
  if (p.act && !(can_asm && lay.a_kc && pr.out_dtype == pr.in_dtype && (p.N & 127) == 0)) return GMM_ERR_UNSUPPORTED;
  if (p.gather) {
    // the assembly tile gathers rows of a K-contiguous first operand whose byte offsets fit 31 bits; the
    // register-staged MFMA kernel has no gather: everything else goes to the generic family
    if (can_asm && !(lay.a_kc && int64_t(p.a_rows) * p.a_sm * 2 < (int64_t(1) << 31))) can_asm = false;
  }
  // fp16 has the assembly tile only (configuration 1); bf16 also the register-staged kernel
  const bool can_mfma = aligned && (p.gather ? can_asm : (pr.in_dtype == GMM_DT_BF16 || can_asm));
  if (forced == GMM_PATH_MFMA && !can_mfma) return GMM_ERR_UNSUPPORTED;
  const bool use_mfma = can_mfma && forced != GMM_PATH_GENERIC;

  int rc;
  if (use_mfma) {
    p.align = align;
    p.xcd_remap = g_xcd_remap.load(std::memory_order_relaxed);
    int cfg = g_forced_config.load(std::memory_order_relaxed);
    if (cfg == GMM_CFG_ASM_256x256 && !can_asm) return GMM_ERR_UNSUPPORTED;
    if (cfg < 0 || cfg >= GMM_CFG_COUNT) cfg = can_asm ? GMM_CFG_ASM_256x256 : GMM_CFG_REG_256x256;
    if ((p.gather || p.act) && cfg != GMM_CFG_ASM_256x256) return GMM_ERR_UNSUPPORTED;
    if (pr.in_dtype != GMM_DT_BF16 && cfg != GMM_CFG_ASM_256x256) return GMM_ERR_UNSUPPORTED;
    // the assembly tile stores 16-byte chunks: its tile columns start at multiples of 8 elements
    if (cfg == GMM_CFG_ASM_256x256 && p.jag == GMM_JAG_N) p.align = 8;
    // Tile heights of the assembly tile: 256-row tiles unless the launch would not even fill four rounds
    // of the grid, then 128; 64-row tiles for group remainders whenever A is contiguous along K.
    {
      const int64_t tn = (p.N + 255) / 256;
      int64_t est = int64_t(p.G) * ((p.M + 255) / 256) * tn;
      if (p.jag == GMM_JAG_M) est = (int64_t(p.M) / 256 + (p.G < p.M ? p.G : p.M)) * tn;
      if (p.jag == GMM_JAG_N) est = (int64_t(p.N) / 256 + (p.G < p.N ? p.G : p.N)) * ((p.M + 255) / 256);
      p.tall = (lay.a_kc && est < 4 * int64_t(cus)) ? 128 : 256;
      p.shrt = lay.a_kc ? 64 : 0;
      const int ft = g_forced_tall.load(std::memory_order_relaxed), fs = g_forced_short.load(std::memory_order_relaxed);
      if (lay.a_kc && (ft == 256 || ft == 128)) p.tall = ft;
      if (lay.a_kc && (fs == 0 || fs == 64)) p.shrt = fs;
    }
    // Launch order: group by group in the fine-grained regime (many small groups: a group's remainder tile
    // then reads the second operand while its tall tiles have it in the caches; +4 % there), otherwise all
    // tall tiles first (longest first balances the rounds; the down projection loses 1 % group by group).
    {
      const int fo = g_group_major.load(std::memory_order_relaxed);
      p.group_major = fo >= 0 ? fo : (p.tall == 128 ? 1 : 0);
    }
    rc = gmm_launch_mfma(p, lay, pr.in_dtype, pr.out_dtype, cfg, cus, stream);
    t_last_path = GMM_PATH_MFMA;
    t_last_config = cfg;
  } else {
    rc = gmm_launch_generic(p, pr.in_dtype, pr.out_dtype, cus, stream);
    t_last_path = GMM_PATH_GENERIC;
    t_last_config = -1;
  }
  if (rc < 0) return GMM_ERR_UNSUPPORTED;
  return rc == 0 ? GMM_OK : GMM_ERR_LAUNCH;
}

bool dims_ok(int64_t a, int64_t b, int64_t c) { return fits_i32(a) && fits_i32(b) && fits_i32(c); }

}  // namespace

extern "C" {

int gmm_abi_version(void) { return GMM_ABI_VERSION; }

int64_t gmm_workspace_bytes(void) {
  const int cus = device_cus();
  return cus > 0 ? GMM_WS_HEADER + 2 * int64_t(cus) * GMM_WS_SLOT : 0;
}

const char* gmm_status_string(int status) {
  switch (status) {
    case GMM_OK: return "ok";
    case GMM_ERR_BAD_ARGUMENT: return "bad argument (null pointer, size out of range or more than 1023 groups)";
    case GMM_ERR_UNSUPPORTED: return "unsupported dtype combination or forced kernel family not applicable";
    case GMM_ERR_LAUNCH: return "HIP launch failed";
    case GMM_ERR_WORKSPACE: return "workspace too small for this problem";
    default: return "unknown status";
  }
}

int gmm_2d3d(const void* a, const void* b, void* out, const int32_t* offs, int32_t G, int64_t M_total,
             int64_t N, int64_t K, int64_t a_sm, int64_t a_sk, int64_t b_sg, int64_t b_sk, int64_t b_sn,
             int64_t o_sm, int64_t o_sn, int32_t in_dtype, int32_t out_dtype, void* workspace,
             int64_t workspace_bytes, void* stream) {
  if (!dims_ok(M_total, N, K)) return GMM_ERR_BAD_ARGUMENT;
  Problem pr{};
  pr.p = GmmParams{a, b, out, offs, G, GMM_JAG_M, int32_t(M_total), int32_t(N), int32_t(K), 1,
                   0, a_sm, a_sk, b_sg, b_sk, b_sn, 0, o_sm, o_sn, 0, 0};
  pr.in_dtype = in_dtype;
  pr.out_dtype = out_dtype;
  set_workspace(pr.p, workspace, workspace_bytes);
  return run(pr, static_cast<hipStream_t>(stream));
}

int gmm_2d3d_gather(const void* a, const int32_t* row_index, const void* b, void* out, const int32_t* offs, int32_t G,
                    int64_t a_rows, int64_t M_total, int64_t N, int64_t K, int64_t a_sm, int64_t a_sk, int64_t b_sg,
                    int64_t b_sk, int64_t b_sn, int64_t o_sm, int64_t o_sn, int32_t in_dtype, int32_t out_dtype, void* workspace,
                    int64_t workspace_bytes, void* stream) {
  if (!dims_ok(M_total, N, K) || !fits_i32(a_rows)) return GMM_ERR_BAD_ARGUMENT;
  if (!row_index && M_total > 0 && G > 0 && N > 0) return GMM_ERR_BAD_ARGUMENT;
  Problem pr{};
  pr.p = GmmParams{a, b, out, offs, G, GMM_JAG_M, int32_t(M_total), int32_t(N), int32_t(K), 1,
                   0, a_sm, a_sk, b_sg, b_sk, b_sn, 0, o_sm, o_sn, 0, 0};
  pr.p.gather = row_index;
  pr.p.a_rows = int32_t(a_rows);
  pr.in_dtype = in_dtype;
  pr.out_dtype = out_dtype;
  set_workspace(pr.p, workspace, workspace_bytes);
  return run(pr, static_cast<hipStream_t>(stream));
}

int gmm_2d3d_swiglu(const void* a, const int32_t* row_index, const void* b, void* out, const int32_t* offs, int32_t G,
                    int64_t a_rows, int64_t M_total, int64_t N, int64_t K, int64_t a_sm, int64_t a_sk, int64_t b_sg,
                    int64_t b_sk, int64_t b_sn, int64_t o_sm, int64_t o_sn, int32_t dtype, void* stream) {
  if (!dims_ok(M_total, N, K) || !fits_i32(a_rows)) return GMM_ERR_BAD_ARGUMENT;
  Problem pr{};
  pr.p = GmmParams{a, b, out, offs, G, GMM_JAG_M, int32_t(M_total), int32_t(N), int32_t(K), 1,
                   0, a_sm, a_sk, b_sg, b_sk, b_sn, 0, o_sm, o_sn, 0, 0};
  pr.p.gather = row_index;
  pr.p.a_rows = int32_t(row_index ? a_rows : M_total);
  pr.p.act = 1;
  pr.in_dtype = dtype;
  pr.out_dtype = dtype;
  if (g_forced_path.load(std::memory_order_relaxed) == GMM_PATH_GENERIC) return GMM_ERR_UNSUPPORTED;
  return run(pr, static_cast<hipStream_t>(stream));
}

int gmm_3d3d(const void* a, const void* b, void* out, int32_t G, int64_t M, int64_t N, int64_t K,
             int64_t a_sg, int64_t a_sm, int64_t a_sk, int64_t b_sg, int64_t b_sk, int64_t b_sn,
             int64_t o_sg, int64_t o_sm, int64_t o_sn, int32_t in_dtype, int32_t out_dtype, void* workspace,
             int64_t workspace_bytes, void* stream) {
  if (!dims_ok(M, N, K)) return GMM_ERR_BAD_ARGUMENT;
  Problem pr{};
  pr.p = GmmParams{a, b, out, nullptr, G, GMM_JAG_NONE, int32_t(M), int32_t(N), int32_t(K), 1,
                   a_sg, a_sm, a_sk, b_sg, b_sk, b_sn, o_sg, o_sm, o_sn, 0, 0};
  pr.in_dtype = in_dtype;
  pr.out_dtype = out_dtype;
  set_workspace(pr.p, workspace, workspace_bytes);
  // the tile count G * tiles must fit an int32
  if (G > 0 && M > 0 && N > 0) {
    const int64_t tiles = int64_t(G) * ((M + 63) / 64) * ((N + 63) / 64);
    if (!fits_i32(tiles)) return GMM_ERR_BAD_ARGUMENT;
  }
  return run(pr, static_cast<hipStream_t>(stream));
}

int gmm_2d2d(const void* a, const void* b, void* out, const int32_t* offs, int32_t G, int64_t M, int64_t N,
             int64_t K_total, int64_t a_sm, int64_t a_sk, int64_t b_sk, int64_t b_sn, int64_t o_sg,
             int64_t o_sm, int64_t o_sn, int32_t in_dtype, int32_t out_dtype, void* workspace,
             int64_t workspace_bytes, void* stream) {
  if (!dims_ok(M, N, K_total)) return GMM_ERR_BAD_ARGUMENT;
  Problem pr{};
  pr.p = GmmParams{a, b, out, offs, G, GMM_JAG_K, int32_t(M), int32_t(N), int32_t(K_total), 1,
                   0, a_sm, a_sk, 0, b_sk, b_sn, o_sg, o_sm, o_sn, 0, 0};
  pr.in_dtype = in_dtype;
  pr.out_dtype = out_dtype;
  set_workspace(pr.p, workspace, workspace_bytes);
  return run(pr, static_cast<hipStream_t>(stream));
}

int gmm_3d2d(const void* a, const void* b, void* out, const int32_t* offs, int32_t G, int64_t M,
             int64_t N_total, int64_t K, int64_t a_sg, int64_t a_sm, int64_t a_sk, int64_t b_sk, int64_t b_sn,
             int64_t o_sm, int64_t o_sn, int32_t in_dtype, int32_t out_dtype, void* workspace,
             int64_t workspace_bytes, void* stream) {
  if (!dims_ok(M, N_total, K)) return GMM_ERR_BAD_ARGUMENT;
  Problem pr{};
  pr.p = GmmParams{a, b, out, offs, G, GMM_JAG_N, int32_t(M), int32_t(N_total), int32_t(K), 1,
                   a_sg, a_sm, a_sk, 0, b_sk, b_sn, 0, o_sm, o_sn, 0, 0};
  pr.in_dtype = in_dtype;
  pr.out_dtype = out_dtype;
  set_workspace(pr.p, workspace, workspace_bytes);
  return run(pr, static_cast<hipStream_t>(stream));
}

int gmm_set_path(int path) {
  if (path < GMM_PATH_AUTO || path > GMM_PATH_MFMA) return -1;
  return g_forced_path.exchange(path);
}
int gmm_last_path(void) { return t_last_path; }
int gmm_set_mfma_config(int config) { return g_forced_config.exchange(config); }
int gmm_last_mfma_config(void) { return t_last_config; }
int gmm_set_xcd_remap(int on) { return g_xcd_remap.exchange(on ? 1 : 0); }
int gmm_set_group_major(int mode) { return g_group_major.exchange(mode < 0 ? -1 : (mode ? 1 : 0)); }
int gmm_set_tail_split(int on) { return g_tail_split.exchange(on ? 1 : 0); }
int gmm_set_tile_heights(int tall, int shrt) {
  const int prev_tall = g_forced_tall.exchange(tall), prev_short = g_forced_short.exchange(shrt);
  return ((prev_tall + 1) << 16) | ((prev_short + 1) & 0xffff);
}

int64_t gmm_host_tile_list(const int32_t* offs_host, int32_t G, int32_t jagged, int32_t M, int32_t N, int32_t K,
                           int32_t tile_m, int32_t tile_n, int32_t align, int32_t xcd_remap,
                           int32_t num_workgroups, int32_t* records, int64_t capacity) {
  if (G < 0 || jagged < 0 || jagged > 3 || tile_m <= 0 || tile_n <= 0 || align <= 0) return -GMM_ERR_BAD_ARGUMENT;
  if (jagged != GMM_JAG_NONE && (!offs_host || G < 1 || G >= GMM_MAX_GROUPS)) return -GMM_ERR_BAD_ARGUMENT;
  if (xcd_remap && (num_workgroups <= 0 || num_workgroups % 8)) return -GMM_ERR_BAD_ARGUMENT;
  GmmParams p{};
  p.offs = offs_host;
  p.G = G; p.jag = jagged; p.M = M; p.N = N; p.K = K; p.align = align;
  const int extent = jagged == GMM_JAG_M ? M : (jagged == GMM_JAG_N ? N : K);
  std::vector<int32_t> cum(size_t(G) + 1, 0);
  for (int g = 0; g < G; ++g) {
    int lo = 0, hi = 0, tm, tn;
    if (jagged != GMM_JAG_NONE) gmm_group_range(offs_host, g, extent, lo, hi);
    gmm_group_grid(jagged, lo, hi, M, N, tile_m, tile_n, align, tm, tn);
    cum[g + 1] = cum[g] + tm * tn;
  }
  const int total = cum[G];
  for (int t = 0; t < total; ++t) {
    const int tt = xcd_remap ? gmm_xcd_remap(t, total, num_workgroups) : t;
    const int g = gmm_find_group(cum.data(), G, tt);
    int lo = 0, hi = 0, tm, tn, mt, nt;
    if (jagged != GMM_JAG_NONE) gmm_group_range(offs_host, g, extent, lo, hi);
    gmm_group_grid(jagged, lo, hi, M, N, tile_m, tile_n, align, tm, tn);
    gmm_decode_in_group(tt - cum[g], tm, tn, mt, nt);
    const GmmTile tile = gmm_make_tile(p, g, lo, hi, mt, nt, tile_m, tile_n);
    if (t < capacity && records) {
      int32_t* r = records + int64_t(t) * 9;
      r[0] = tile.g; r[1] = tile.m0; r[2] = tile.n0; r[3] = tile.m_lo; r[4] = tile.m_hi;
      r[5] = tile.n_lo; r[6] = tile.n_hi; r[7] = tile.k_lo; r[8] = tile.k_hi;
    }
  }
  return total;
}

// Shared by gmm_host_tile_list2 / 3: the launch order of the assembly tile's kernel, run on the host.
static int64_t host_tile_list23(const int32_t* offs_host, int32_t G, int32_t jagged, int32_t M, int32_t N, int32_t K,
                                int32_t tall, int32_t shrt, int32_t tile_n, int32_t align, int32_t xcd_remap,
                                int32_t num_workgroups, int32_t max_parts, int32_t group_major, int32_t width,
                                int32_t* records, int64_t capacity) {
  if (G < 0 || jagged < 0 || jagged > 3 || tall <= 0 || shrt < 0 || tile_n <= 0 || align <= 0 || max_parts < 0)
    return -GMM_ERR_BAD_ARGUMENT;
  if (jagged != GMM_JAG_NONE && (!offs_host || G < 1 || G >= GMM_MAX_GROUPS)) return -GMM_ERR_BAD_ARGUMENT;
  if ((xcd_remap || max_parts) && (num_workgroups <= 0 || num_workgroups % 8)) return -GMM_ERR_BAD_ARGUMENT;
  GmmParams p{};
  p.offs = offs_host;
  p.G = G; p.jag = jagged; p.M = M; p.N = N; p.K = K; p.align = align; p.tall = tall; p.shrt = shrt;
  const int extent = jagged == GMM_JAG_M ? M : (jagged == GMM_JAG_N ? N : K);
  std::vector<int32_t> ct(size_t(G) + 1, 0), cs(size_t(G) + 1, 0);
  for (int g = 0; g < G; ++g) {
    int lo = 0, hi = 0, n_tall, n_short, rem_rows;
    if (jagged != GMM_JAG_NONE) gmm_group_range(offs_host, g, extent, lo, hi);
    gmm_split_rows(gmm_group_rows(jagged, lo, hi, M, align), tall, shrt, n_tall, n_short, rem_rows);
    const int tn = gmm_group_tile_cols(jagged, lo, hi, N, align, tile_n);
    ct[g + 1] = ct[g] + n_tall * tn + (group_major ? n_short * tn : 0);
    cs[g + 1] = cs[g] + (group_major ? 0 : n_short * tn);
  }
  const int total_tall = ct[G], total_tiles = ct[G] + cs[G];
  // the split of the last round, as gmm_asm_kernel decides it
  const int nk = gmm_cdiv(K, 64);
  int nparts = 1, tail = 0;
  if (max_parts > 0 && jagged != GMM_JAG_K) {
    nparts = gmm_tail_split(total_tiles, num_workgroups, nk, max_parts);
    if (nparts > 1) tail = total_tiles % num_workgroups;
  }
  // round-robin tiles in launch order, then the parts in ticket order (which workgroup runs a part is
  // decided at run time)
  const int split_base = total_tiles - tail, total = split_base + tail * nparts;
  for (int t = 0; t < total; ++t) {
    int tt, part = 0;
    const bool is_part = t >= split_base;
    if (!is_part) {
      tt = xcd_remap ? gmm_xcd_remap(t, split_base, num_workgroups) : t;
    } else {
      part = (t - split_base) / tail;
      tt = split_base + (t - split_base) % tail;
    }
    int cls = tt < total_tall ? 0 : 1;
    const int tc = cls ? tt - total_tall : tt;
    const std::vector<int32_t>& cum = cls ? cs : ct;
    const int g = gmm_find_group(cum.data(), G, tc);
    int lo = 0, hi = 0, local = tc - cum[g];
    if (jagged != GMM_JAG_NONE) gmm_group_range(offs_host, g, extent, lo, hi);
    if (group_major) {
      // one table: a group's tall tiles, then its remainder tiles
      int n_tall, n_short, rem_rows;
      gmm_split_rows(gmm_group_rows(jagged, lo, hi, M, align), tall, shrt, n_tall, n_short, rem_rows);
      const int tall_tiles = n_tall * gmm_group_tile_cols(jagged, lo, hi, N, align, tile_n);
      if (local >= tall_tiles) { cls = 1; local -= tall_tiles; }
    }
    GmmTile tile = gmm_make_tile2(p, g, lo, hi, cls, local, tile_n);
    if (is_part) {
      int kt0, kt1;
      gmm_part_ktiles(nk, nparts, part, kt0, kt1);
      tile.k_lo = kt0 * 64;
      tile.k_hi = gmm_min(kt1 * 64, K);
    }
    if (t < capacity && records) {
      int32_t* r = records + int64_t(t) * width;
      r[0] = tile.g; r[1] = tile.m0; r[2] = tile.n0; r[3] = tile.m_lo; r[4] = tile.m_hi;
      r[5] = tile.n_lo; r[6] = tile.n_hi; r[7] = tile.k_lo; r[8] = tile.k_hi; r[9] = tile.rows;
      if (width >= 12) { r[10] = part; r[11] = is_part ? nparts : 1; }
    }
  }
  return total;
}

int64_t gmm_host_tile_list2(const int32_t* offs_host, int32_t G, int32_t jagged, int32_t M, int32_t N, int32_t K,
                            int32_t tall, int32_t shrt, int32_t tile_n, int32_t align, int32_t xcd_remap,
                            int32_t num_workgroups, int32_t* records, int64_t capacity) {
  return host_tile_list23(offs_host, G, jagged, M, N, K, tall, shrt, tile_n, align, xcd_remap, num_workgroups, 0, 0, 10,
                          records, capacity);
}

int64_t gmm_host_tile_list3(const int32_t* offs_host, int32_t G, int32_t jagged, int32_t M, int32_t N, int32_t K,
                            int32_t tall, int32_t shrt, int32_t tile_n, int32_t align, int32_t xcd_remap,
                            int32_t num_workgroups, int32_t max_parts, int32_t group_major, int32_t* records,
                            int64_t capacity) {
  if (group_major && jagged == GMM_JAG_NONE) group_major = 0;   // batches are all alike: one order
  return host_tile_list23(offs_host, G, jagged, M, N, K, tall, shrt, tile_n, align, xcd_remap, num_workgroups,
                          max_parts, group_major ? 1 : 0, 12, records, capacity);
}

}  // extern "C"
