/* C ABI of libgrouped_mm_hip.so: grouped matrix multiply for AMD MI355X (gfx950).
 *
 * The four launchers replace, one for one, the forward launchers that the
 * reference's host layer imports (reference grouped_mm_bf16/api.py:8-17) and
 * calls at api.py:195, 201, 207 and 213.  Like them they write into an output the
 * caller allocated, return without synchronising, and never allocate.
 *
 * Conventions
 *   - all pointers are device pointers on the current HIP device;
 *   - strides are in ELEMENTS, one per tensor dimension, exactly torch's
 *     tensor.stride(); every operand may be row-major or column-major in its
 *     last two dimensions, with any batch stride and any alignment;
 *   - `offs` is int32[G] of non-decreasing END offsets along the jagged
 *     dimension (the first group starts at 0); it is read on the device only;
 *   - in_dtype / out_dtype are gmm_dtype values; out_dtype is in_dtype or
 *     GMM_DT_F32;
 *   - `workspace` / `workspace_bytes`: optional device memory (NULL / 0: none) that lets a launch whose
 *     last round of tiles would leave most of the chip idle cut those tiles along the contraction (see
 *     gmm_workspace_bytes below); the library itself never allocates;
 *   - `stream` is a hipStream_t (NULL = the default stream);
 *   - the return value is a gmm_status; nothing is thrown across the boundary.
 *   - elements that no group owns (rows / columns at or beyond offs[G-1]) are
 *     not written; with G == 0 nothing is written and GMM_OK is returned.
 */
#ifndef GROUPED_MM_HIP_H
#define GROUPED_MM_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GMM_ABI_VERSION 3

enum gmm_status {
  GMM_OK = 0,
  GMM_ERR_BAD_ARGUMENT = 1, /* null pointer, negative size, G out of range, bad stride */
  GMM_ERR_UNSUPPORTED = 2,  /* dtype combination or forced path not available */
  GMM_ERR_LAUNCH = 3,       /* the HIP runtime refused the launch */
  GMM_ERR_WORKSPACE = 4     /* the workspace passed in is smaller than the problem needs */
};

enum gmm_dtype { GMM_DT_BF16 = 0, GMM_DT_F16 = 1, GMM_DT_F32 = 2 };

/* Kernel families.  AUTO picks MFMA when the operands qualify (bf16 or fp16, 16-byte
 * aligned bases and leading dimensions), else GENERIC. */
enum gmm_path { GMM_PATH_AUTO = 0, GMM_PATH_GENERIC = 1, GMM_PATH_MFMA = 2 };

int gmm_abi_version(void);
const char* gmm_status_string(int status);

/* Workspace of the launchers below.  The kernels deal output tiles to one workgroup per compute unit, round
 * by round; when the last round holds far fewer tiles than there are compute units (a down projection
 * 16384 x 14336 -> 4096 has 4.25 rounds of tiles on 256 units) its tiles are cut along the contraction into
 * up to 8 parts, every part stores an fp32 partial tile in the workspace, and the part that arrives last adds
 * the partials in part order and stores the output: the result does not depend on timing and is rounded
 * once.  Layout: 4096 bytes of arrival counters, then slots of 262144 bytes (one fp32 tile each); the more
 * slots, the more freedom to split.  gmm_workspace_bytes() returns the size the library can make full use
 * of on the current device (4096 + 2 * compute units * 262144; 128 MiB on MI355X); a smaller workspace
 * limits the split, less than 4096 + 2 * 262144 bytes (or NULL) turns it off.  Rules for the caller:
 *   - 16-byte aligned; the first 4096 bytes zero before the first launch that uses it (the kernels leave
 *     them zero, so one hipMemset after allocation is enough); the rest need not be initialised;
 *   - launches that may run at the same time (different streams) need different workspaces.
 * The reference has no counterpart (its launches create one program per tile, reference
 * kernels.py:636-659, and leave the balancing to the hardware dispatcher). */
int64_t gmm_workspace_bytes(void);

/* 2D x 3D: out[s_g:e_g, :] = a[s_g:e_g, :] @ b[g]   (rows jagged)
 * a [M_total, K], b [G, K, N], out [M_total, N].
 * Replaces grouped_mm_2d3d(mat_a, mat_b, offs, out), reference kernels.py:583-686. */
int gmm_2d3d(const void* a, const void* b, void* out, const int32_t* offs, int32_t G,
             int64_t M_total, int64_t N, int64_t K,
             int64_t a_stride_m, int64_t a_stride_k,
             int64_t b_stride_g, int64_t b_stride_k, int64_t b_stride_n,
             int64_t out_stride_m, int64_t out_stride_n,
             int32_t in_dtype, int32_t out_dtype,
             void* workspace, int64_t workspace_bytes, void* stream);

/* 2D x 3D with the rows of the first operand gathered on the fly:
 *   out[r, :] = a[row_index[r], :] @ b[g(r)]   for r < offs[G-1], g(r) the group that owns row r.
 * a [a_rows, K], row_index int32[M_total] (device), b [G, K, N], out [M_total, N].  An index outside
 * [0, a_rows) reads a row of zeros.  This is gmm_2d3d applied to a[row_index] without materialising the
 * permuted copy: the token gather that a mixture-of-experts layer performs between routing and the up
 * projection (the reference's benchmark starts from rows already sorted, bench/bench_2d3d.py:140-149).
 * The assembly tile takes it when `a` is contiguous along K and a_rows * a_stride_m * 2 < 2^31. */
int gmm_2d3d_gather(const void* a, const int32_t* row_index, const void* b, void* out,
                    const int32_t* offs, int32_t G, int64_t a_rows,
                    int64_t M_total, int64_t N, int64_t K,
                    int64_t a_stride_m, int64_t a_stride_k,
                    int64_t b_stride_g, int64_t b_stride_k, int64_t b_stride_n,
                    int64_t out_stride_m, int64_t out_stride_n,
                    int32_t in_dtype, int32_t out_dtype,
                    void* workspace, int64_t workspace_bytes, void* stream);

/* 2D x 3D with the SwiGLU activation applied to the product before it is stored (and, optionally, the row
 * gather above: row_index may be NULL for rows already in place, a_rows is then ignored).
 * b [G, K, N] holds, in every block of 128 columns, 64 gate columns followed by their 64 partner columns:
 *   h = a[row_index] @ b[g]  (fp32),   out[r, 64 * blk + c] = silu(h[r, 128 * blk + c]) * h[r, 128 * blk + 64 + c],
 * out [M_total, N / 2] in the input dtype (bf16 or fp16), rounded once: the intermediate h is never written.
 * Assembly tile only: returns GMM_ERR_UNSUPPORTED unless a is contiguous along K, N % 128 == 0 and the
 * operands meet the alignment rules of the fast path (16-byte aligned bases, leading dimensions multiples of
 * 8 elements, out row-major).  No counterpart in the reference. */
int gmm_2d3d_swiglu(const void* a, const int32_t* row_index, const void* b, void* out,
                    const int32_t* offs, int32_t G, int64_t a_rows,
                    int64_t M_total, int64_t N, int64_t K,
                    int64_t a_stride_m, int64_t a_stride_k,
                    int64_t b_stride_g, int64_t b_stride_k, int64_t b_stride_n,
                    int64_t out_stride_m, int64_t out_stride_n,
                    int32_t dtype, void* stream);

/* 3D x 3D: out[g] = a[g] @ b[g]
 * a [G, M, K], b [G, K, N], out [G, M, N].
 * Replaces grouped_mm_3d3d(mat_a, mat_b, out), reference kernels.py:524-550. */
int gmm_3d3d(const void* a, const void* b, void* out, int32_t G,
             int64_t M, int64_t N, int64_t K,
             int64_t a_stride_g, int64_t a_stride_m, int64_t a_stride_k,
             int64_t b_stride_g, int64_t b_stride_k, int64_t b_stride_n,
             int64_t out_stride_g, int64_t out_stride_m, int64_t out_stride_n,
             int32_t in_dtype, int32_t out_dtype,
             void* workspace, int64_t workspace_bytes, void* stream);

/* 2D x 2D: out[g] = a[:, s_g:e_g] @ b[s_g:e_g, :]   (contraction jagged; zeros if empty)
 * a [M, K_total], b [K_total, N], out [G, M, N].
 * Replaces grouped_mm_2d2d(mat_a, mat_b, offs, out), reference kernels.py:553-580. */
int gmm_2d2d(const void* a, const void* b, void* out, const int32_t* offs, int32_t G,
             int64_t M, int64_t N, int64_t K_total,
             int64_t a_stride_m, int64_t a_stride_k,
             int64_t b_stride_k, int64_t b_stride_n,
             int64_t out_stride_g, int64_t out_stride_m, int64_t out_stride_n,
             int32_t in_dtype, int32_t out_dtype,
             void* workspace, int64_t workspace_bytes, void* stream);

/* 3D x 2D: out[:, s_g:e_g] = a[g] @ b[:, s_g:e_g]   (columns jagged)
 * a [G, M, K], b [K, N_total], out [M, N_total].
 * Replaces grouped_mm_3d2d(mat_a, mat_b, offs, out), reference kernels.py:689-717. */
int gmm_3d2d(const void* a, const void* b, void* out, const int32_t* offs, int32_t G,
             int64_t M, int64_t N_total, int64_t K,
             int64_t a_stride_g, int64_t a_stride_m, int64_t a_stride_k,
             int64_t b_stride_k, int64_t b_stride_n,
             int64_t out_stride_m, int64_t out_stride_n,
             int32_t in_dtype, int32_t out_dtype,
             void* workspace, int64_t workspace_bytes, void* stream);

/* ---- The mixture-of-experts step either side of the grouped product.  The reference has no such code;
 * its benchmark builds the sorted rows and `offs` with torch on the host side (bench/bench_2d3d.py:124-149:
 * randint / bincount / cumsum and an offs[-1].item() round trip).  Here everything stays on the device.
 *
 * Routing.  For each of `tokens` rows of `logits` [tokens, experts] (row stride logits_stride elements,
 * dtype a gmm_dtype) pick the top_k largest (ties: lower expert index first; logits must not be NaN; -inf
 * masks an expert; a row whose maximum is +inf or -inf puts all weight, in equal shares, on the entries equal
 * to the maximum: the limit of the softmax), in
 * descending order.  Choice j of token t is SLOT t * top_k + j.  Outputs (device memory):
 *   slot_expert int32[tokens * top_k]   expert of each slot
 *   slot_weight float[tokens * top_k]   softmax over the token's chosen logits (renormalize != 0), or the
 *                                       chosen entries of the softmax over all experts (renormalize == 0)
 *   offs        int32[experts]          end offsets of the experts' row ranges (inclusive prefix of counts)
 *   row_token   int32[tokens * top_k]   rows sorted by expert, stably in slot order: the token of each row
 *   token_rows  int32[tokens * top_k]   the row of each slot (inverse of the sort)
 * experts <= 1023, top_k <= min(experts, 32), tokens * top_k < 2^31.  `workspace` is device memory of at
 * least gmm_moe_route_workspace_bytes(...) bytes (per-workgroup expert histograms; contents need not be
 * initialised); too small a workspace returns GMM_ERR_WORKSPACE.  Four launches on `stream`, no host sync. */
int64_t gmm_moe_route_workspace_bytes(int64_t tokens, int64_t experts, int64_t top_k);
int gmm_moe_route(const void* logits, int64_t logits_stride, int32_t logits_dtype,
                  int64_t tokens, int64_t experts, int64_t top_k, int32_t renormalize,
                  int32_t* offs, int32_t* slot_expert, float* slot_weight,
                  int32_t* row_token, int32_t* token_rows,
                  void* workspace, int64_t workspace_bytes, void* stream);

/* gmm_moe_route without a workspace argument.  No counterpart in the reference: it is for callers that
 * cannot allocate device memory or pass a workspace around (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  The histogram table lives in a 256 KiB array that the library
 * holds on every GPU it runs on until the process ends; the call allocates nothing.  Problems whose
 * gmm_moe_route_workspace_bytes(...) exceeds 262144 bytes are refused with GMM_ERR_WORKSPACE (any problem
 * with experts <= 256 fits; with 1023 experts up to 65536 slots).  All calls on one GPU share that array:
 * calls that may overlap on one GPU (different streams, different threads) race and must be serialised by
 * the caller.  The first call on a device looks the array's device address up (hipGetSymbolAddress, no
 * allocation): make that first call outside a stream capture -- one eager call per device at start-up is
 * enough -- and every later call, captured or not, only launches.  Outputs and everything else as
 * gmm_moe_route. */
int gmm_moe_route_noalloc(const void* logits, int64_t logits_stride, int32_t logits_dtype,
                          int64_t tokens, int64_t experts, int64_t top_k, int32_t renormalize,
                          int32_t* offs, int32_t* slot_expert, float* slot_weight,
                          int32_t* row_token, int32_t* token_rows, void* stream);

/* Activation between the two projections, bf16 or fp16, fp32 arithmetic and one rounding:
 *   kind 0: out[r, c] = silu(h[r, c]);   kind 1 (SwiGLU): out[r, c] = silu(h[r, c]) * h[r, inner + c],
 * for r < rows, c < inner.  inner and both strides multiples of 8 elements, 16-byte aligned bases. */
int gmm_moe_activation(const void* h, void* out, int64_t rows, int64_t inner,
                       int64_t h_stride, int64_t out_stride, int32_t kind, int32_t dtype, void* stream);

/* Un-permute and weighted sum: out[t, :] = sum_{j < top_k} slot_weight[t * top_k + j] * y[token_rows[t * top_k + j], :],
 * added in fp32 in the order of j and rounded once (no atomics: the result does not depend on timing).
 * y [y_rows, hidden], out [tokens, hidden], bf16 or fp16; hidden and strides multiples of 8, 16-byte aligned
 * bases.  A slot whose row is outside [0, y_rows) contributes nothing. */
int gmm_moe_combine(const void* y, const int32_t* token_rows, const float* slot_weight, void* out,
                    int64_t tokens, int64_t top_k, int64_t hidden, int64_t y_rows,
                    int64_t y_stride, int64_t out_stride, int32_t dtype, void* stream);

/* Test and tuning hooks (the reference exposes its tile knobs through environment
 * variables read in the launcher, kernels.py:590-634; tests force tiles through
 * them, tests/test_grouped_mm.py:388-394).  gmm_set_path forces a kernel family
 * for later calls of this process and returns the previous setting;
 * gmm_last_path reports the family the calling thread's last launch used
 * (GMM_PATH_GENERIC or GMM_PATH_MFMA, 0 before any launch).
 * All gmm_set_* hooks below are process-wide and are not synchronised with launches
 * of other threads (a launch that runs while another thread holds a forced setting
 * takes that setting): they are for tests and tuning runs, not for serving code. */
int gmm_set_path(int path);
int gmm_last_path(void);
/* Tile configuration of the MFMA family: -1 = choose from the shapes, 0 = register-staged kernel,
 * 1 = assembly tile (256 / 128 / 64-row tiles).  Returns the previous setting. */
int gmm_set_mfma_config(int config);
int gmm_last_mfma_config(void);
/* 0 / 1: renumber tiles per XCD (default 1). */
int gmm_set_xcd_remap(int on);
/* Launch order of the assembly tile's kernel: 0 = all tall tiles of all groups, then the remainder tiles;
 * 1 = group by group; -1 (default) = chosen from the shapes (group by group when the tall tiles are 128 rows,
 * the regime of many small groups).  Returns the previous setting. */
int gmm_set_group_major(int mode);
/* 0: later launches ignore their workspace, so no tile is cut along the contraction (tests compare launches
 * bit for bit that would otherwise split differently); 1 (default): use it.  Returns the previous setting. */
int gmm_set_tail_split(int on);
/* Tile heights of the assembly tile: tall = 256 or 128 (-1: chosen from the shapes), shrt = 64 or 0
 * (-1: 64 whenever the first operand is contiguous along the contraction).  Returns the previous
 * setting packed as ((tall + 1) << 16) | (shrt + 1). */
int gmm_set_tile_heights(int tall, int shrt);

/* Host-side run of the tile scheduler that the kernels execute on the device:
 * writes up to `capacity` records of 9 int32 (group, m0, n0, m_lo, m_hi, n_lo,
 * n_hi, k_lo, k_hi) in launch order and returns the number of tiles (which may
 * exceed capacity), or a negative gmm_status.  `offs_host` is a HOST pointer.
 * jagged: 0 none, 1 rows, 2 columns, 3 contraction. */
int64_t gmm_host_tile_list(const int32_t* offs_host, int32_t G, int32_t jagged,
                           int32_t M, int32_t N, int32_t K,
                           int32_t tile_m, int32_t tile_n, int32_t align,
                           int32_t xcd_remap, int32_t num_workgroups,
                           int32_t* records, int64_t capacity);

/* Same for the two-height tile list of the assembly tile (tall tiles first, then 64-row tiles for group
 * remainders): records of 10 int32, the tenth being the tile's height.  jagged: 0, 1 or 3. */
int64_t gmm_host_tile_list2(const int32_t* offs_host, int32_t G, int32_t jagged,
                            int32_t M, int32_t N, int32_t K,
                            int32_t tall, int32_t shrt, int32_t tile_n, int32_t align,
                            int32_t xcd_remap, int32_t num_workgroups,
                            int32_t* records, int64_t capacity);

/* The same list as a launch with a workspace of `max_parts` slots runs it: the tiles of the last, partly
 * filled round cut along the contraction (see gmm_workspace_bytes), listed after the others in the order in
 * which free workgroups draw them.  group_major != 0: the launch order is group by group (a group's tall
 * tiles, then its remainder tiles) instead of all tall tiles first.  Records of 12 int32: the ten above
 * (k_lo / k_hi are the part's range), the part's index and the number of parts of its tile (1: not split). */
int64_t gmm_host_tile_list3(const int32_t* offs_host, int32_t G, int32_t jagged,
                            int32_t M, int32_t N, int32_t K,
                            int32_t tall, int32_t shrt, int32_t tile_n, int32_t align,
                            int32_t xcd_remap, int32_t num_workgroups, int32_t max_parts,
                            int32_t group_major, int32_t* records, int64_t capacity);

#ifdef __cplusplus
}
#endif
#endif /* GROUPED_MM_HIP_H */
