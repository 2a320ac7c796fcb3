// The mixture-of-experts step either side of the grouped product (declared in include/grouped_mm_hip.h):
//   routing   top-k experts per token, their softmax weights, and a stable counting sort of the
//             (token, choice) slots by expert that yields `offs` for the grouped product without the
//             host ever seeing a count (the reference's benchmark does this with bincount / cumsum and an
//             offs[-1].item() round trip, bench/bench_2d3d.py:124-139);
//   activation   SiLU or SwiGLU between the up and the down projection;
//   combine   out[t] = sum_j weight[t, j] * y[row of slot (t, j)], the un-permute, without atomics.
// All of it is HBM- or latency-bound integer / elementwise work: coalesced 16-byte accesses, LDS for the
// histograms and ranks, no matrix cores.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>

#include "../../include/grouped_mm_hip.h"

namespace {

constexpr int kMaxExperts = 1023;        // the grouped product takes fewer than 1024 groups
constexpr int kMaxTopK = 32;
constexpr int kMaxSortBlocks = 256;      // workgroups of the counting sort (rows of the histogram table)
constexpr int kSlotsPerSortBlock = 1024; // aimed-at slots per workgroup
constexpr int kScratchInts = 64 * 1024;  // built-in histogram table of the entry point that allocates nothing

// Histogram table of gmm_moe_route_noalloc: 256 KiB, one copy per GPU, held until the process ends.  In host
// code this name is only a handle for hipGetSymbolAddress; the device address it returns for the current
// device is what the kernels get.  Every entry the kernels read is written earlier in the same call (the
// histogram kernel fills rows 0 .. nb-1 completely), so nothing needs clearing between calls.
static __device__ __align__(256) int32_t scratch[kScratchInts];

constexpr int kMaxDevices = 64;
std::atomic<int32_t*> g_scratch_ptr[kMaxDevices];

// ---------------------------------------------------------------- element types
struct Bf16 { uint16_t bits; };
struct F16 { _Float16 v; };

__device__ __forceinline__ float to_float(Bf16 x) { return __uint_as_float(uint32_t(x.bits) << 16); }
__device__ __forceinline__ float to_float(F16 x) { return float(x.v); }
__device__ __forceinline__ float to_float(float x) { return x; }

template <typename T> __device__ __forceinline__ T from_float(float f);
template <> __device__ __forceinline__ Bf16 from_float<Bf16>(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return Bf16{uint16_t((u >> 16) | 0x40)};   // NaN stays NaN
  u += 0x7fffu + ((u >> 16) & 1u);                                                 // round to nearest even
  return Bf16{uint16_t(u >> 16)};
}
template <> __device__ __forceinline__ F16 from_float<F16>(float f) { return F16{_Float16(f)}; }

template <typename T> struct alignas(16) Vec8 { T v[8]; };

// ---------------------------------------------------------------- wave helpers (64 lanes)
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
  return x;
}
// Maximum over the wave with data-parallel-primitive moves: prefix maxima inside each row of 16 lanes
// (row_shr 1, 2, 4, 8), then lane 15 of a row into the next row (row_bcast15 into rows 1 and 3) and lane 31
// into rows 2 and 3 (row_bcast31); lane 63 ends up with the maximum of all 64.  Lanes a move does not reach
// take 0, the identity.
__device__ __forceinline__ uint32_t wave_umax(uint32_t v) {
#define GMM_DPP_UMAX(ctrl, rows)                                                        \
  {                                                                                     \
    const uint32_t t = uint32_t(__builtin_amdgcn_update_dpp(0, int(v), ctrl, rows, 0xf, false)); \
    v = t > v ? t : v;                                                                  \
  }
  GMM_DPP_UMAX(0x111, 0xf)
  GMM_DPP_UMAX(0x112, 0xf)
  GMM_DPP_UMAX(0x114, 0xf)
  GMM_DPP_UMAX(0x118, 0xf)
  GMM_DPP_UMAX(0x142, 0xa)
  GMM_DPP_UMAX(0x143, 0xc)
#undef GMM_DPP_UMAX
  return uint32_t(__builtin_amdgcn_readlane(int(v), 63));
}

// fp32 -> uint32 whose unsigned order is the numeric order (NaN with a clear sign bit sorts above +inf)
__device__ __forceinline__ uint32_t order_key(float v) {
  const uint32_t u = __float_as_uint(v + 0.0f);   // -0 becomes +0: the two compare equal
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// ---------------------------------------------------------------- routing 1/4: top-k and weights
// One wave per token.  Choice j of token t is slot t * k + j.  Ties go to the lower expert index (a stable
// descending sort).  weight = softmax over the chosen k logits (renorm) or over all E logits.
template <typename T>
__global__ void __launch_bounds__(256) moe_topk_kernel(const T* __restrict__ logits, int64_t ld, int tokens, int E, int k,
                                                       int renorm, int32_t* __restrict__ slot_expert,
                                                       float* __restrict__ slot_weight) {
  __shared__ uint32_t keys[4][1024];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t = blockIdx.x * 4 + wave;
  if (t >= tokens) return;
  const T* row = logits + int64_t(t) * ld;
  uint32_t* kw = keys[wave];   // lane l reads and writes entries l, l + 64, ... only
  for (int e = lane; e < E; e += 64) kw[e] = order_key(to_float(row[e]));
  uint32_t taken = 0, my_key = 0, top_key = 0;
  int my_e = 0;
  const int per_lane = (E + 63) >> 6;
  for (int j = 0; j < k; ++j) {
    // this lane's best entry that is still free (lowest index among equals), then the wave's best key
    uint32_t best = 0;
    int best_i = -1;
    for (int i = 0; i < per_lane; ++i) {
      const int e = lane + (i << 6);
      if (e < E && !((taken >> i) & 1u) && (best_i < 0 || kw[e] > best)) { best = kw[e]; best_i = i; }
    }
    const uint32_t key_win = wave_umax(best_i >= 0 ? best : 0u);
    // lowest expert index among the lanes that hold that key: lowest i first, then lowest lane
    int e_win = 0;
    for (int i = 0; i < per_lane; ++i) {
      const uint64_t holders = __ballot(best_i == i && best == key_win);
      if (holders) { e_win = (i << 6) + __ffsll((unsigned long long)holders) - 1; break; }
    }
    if ((e_win & 63) == lane) taken |= 1u << (e_win >> 6);
    if (lane == j) { my_e = e_win; my_key = key_win; }
    if (j == 0) top_key = key_win;
  }
  // exp(x - m) with an infinite maximum m (a +inf logit, or a row of -inf: every expert masked) is the limit
  // of the softmax: all weight, in equal shares, on the entries that equal the maximum (inf - inf is NaN)
  const float m = key_value(top_key);
  const bool inf_max = (__float_as_uint(m) & 0x7fffffffu) == 0x7f800000u;
  const float p = lane < k ? (inf_max ? (my_key == top_key ? 1.0f : 0.0f) : __expf(key_value(my_key) - m)) : 0.0f;
  float den;
  if (renorm) {
    den = wave_sum(p);
  } else {
    float s = 0.0f;
    for (int e = lane; e < E; e += 64) s += inf_max ? (kw[e] == top_key ? 1.0f : 0.0f) : __expf(key_value(kw[e]) - m);
    den = wave_sum(s);
  }
  if (lane < k) {
    slot_expert[int64_t(t) * k + lane] = my_e;
    slot_weight[int64_t(t) * k + lane] = p / den;
  }
}

// ---------------------------------------------------------------- routing 2/4: per-workgroup histograms
// Workgroup b counts the experts of slots [b * spb, (b + 1) * spb) into row b of the table.
__global__ void __launch_bounds__(256) moe_hist_kernel(const int32_t* __restrict__ slot_expert, int slots, int spb, int E,
                                                       int32_t* __restrict__ table) {
  __shared__ int32_t hist[1024];
  for (int e = threadIdx.x; e < E; e += 256) hist[e] = 0;
  __syncthreads();
  const int s0 = blockIdx.x * spb, s1 = min(slots, s0 + spb);
  for (int s = s0 + threadIdx.x; s < s1; s += 256) atomicAdd(&hist[slot_expert[s]], 1);
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 256) table[int64_t(blockIdx.x) * E + e] = hist[e];
}

// ---------------------------------------------------------------- routing 3/4: column scan + offs
// One workgroup of 1024 threads, thread e owns expert e: the table's column e becomes its exclusive prefix
// over the workgroups, and offs[e] the inclusive prefix of the expert totals.
__global__ void __launch_bounds__(1024) moe_scan_kernel(int32_t* __restrict__ table, int nb, int E, int32_t* __restrict__ offs) {
  __shared__ int32_t part[16];
  const int e = threadIdx.x, lane = e & 63, wave = e >> 6;
  int run = 0;
  if (e < E) {
    // eight independent loads at a time (each costs a trip to L2), then their exclusive prefixes
    for (int b0 = 0; b0 < nb; b0 += 8) {
      int c[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) c[i] = b0 + i < nb ? table[int64_t(b0 + i) * E + e] : 0;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (b0 + i < nb) table[int64_t(b0 + i) * E + e] = run;
        run += c[i];
      }
    }
  }
  int incl = run;   // inclusive scan of `run` over the 1024 threads
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int up = __shfl_up(incl, o);
    if (lane >= o) incl += up;
  }
  if (lane == 63) part[wave] = incl;
  __syncthreads();
  int base = 0;
  for (int w = 0; w < wave; ++w) base += part[w];
  if (e < E) offs[e] = base + incl;
}

// ---------------------------------------------------------------- routing 4/4: stable scatter
// Workgroup b (one wave) places its slots, in slot order, behind what earlier workgroups hold of the same
// expert: row = offs[e - 1] + (slots of expert e in earlier workgroups) + (earlier slots of e in this one).
// 64 slots at a time: the lanes that hold the same expert find each other with one ballot per bit of the
// expert index, and a lane's rank among them is the population count of the lower lanes in that set.
__global__ void __launch_bounds__(64) moe_scatter_kernel(const int32_t* __restrict__ slot_expert, int slots, int spb, int E,
                                                         int k, const int32_t* __restrict__ table,
                                                         const int32_t* __restrict__ offs, int32_t* __restrict__ row_token,
                                                         int32_t* __restrict__ token_rows) {
  __shared__ int32_t cursor[1024];
  const int lane = threadIdx.x;
  for (int e = lane; e < E; e += 64) cursor[e] = table[int64_t(blockIdx.x) * E + e] + (e ? offs[e - 1] : 0);
  __syncthreads();
  const int s0 = blockIdx.x * spb, s1 = min(slots, s0 + spb);
  const int bits = E > 1 ? 32 - __clz(E - 1) : 0;   // bits that can differ between expert indices
  const uint64_t lower = (uint64_t(1) << lane) - 1;
  for (int c4 = s0; c4 < s1; c4 += 256) {
    int ev[4];   // four chunks' loads in flight at once: each is a trip to L2 or further
#pragma unroll
    for (int i = 0; i < 4; ++i) ev[i] = c4 + 64 * i + lane < s1 ? slot_expert[c4 + 64 * i + lane] : -1;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int s = c4 + 64 * i + lane, e = ev[i];
      const bool live = e >= 0;
      if (c4 + 64 * i >= s1) break;   // uniform
      uint64_t same = __ballot(live);
      for (int bit = 0; bit < bits; ++bit) {
        const bool on = (e >> bit) & 1;
        const uint64_t with_bit = __ballot(on && live);
        same &= on ? with_bit : ~with_bit;
      }
      const int before = __popcll(same & lower), total = __popcll(same);
      int row = 0;
      if (live) row = cursor[e] + before;
      __syncthreads();   // every lane has read its cursor
      if (live) {
        if (before == total - 1) cursor[e] += total;
        row_token[row] = s / k;
        token_rows[s] = row;
      }
      __syncthreads();
    }
  }
}

// ---------------------------------------------------------------- activation
// kind 0: out = silu(h);  kind 1: out = silu(h[:, :inner]) * h[:, inner:2 * inner].  fp32 arithmetic, one
// rounding.  Each thread handles 8 adjacent elements (16 bytes).
template <typename T>
__global__ void __launch_bounds__(256) moe_act_kernel(const T* __restrict__ h, T* __restrict__ out, int64_t rows, int64_t inner,
                                                      int64_t ld_h, int64_t ld_out, int kind) {
  const int64_t vec_per_row = inner >> 3, total = rows * vec_per_row;
  for (int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x; i < total; i += int64_t(gridDim.x) * 256) {
    const int64_t r = i / vec_per_row, c = (i - r * vec_per_row) << 3;
    const Vec8<T> g = *reinterpret_cast<const Vec8<T>*>(h + r * ld_h + c);
    Vec8<T> u, o;
    if (kind) u = *reinterpret_cast<const Vec8<T>*>(h + r * ld_h + inner + c);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float x = to_float(g.v[j]);
      float y = x / (1.0f + __expf(-x));
      if (kind) y *= to_float(u.v[j]);
      o.v[j] = from_float<T>(y);
    }
    *reinterpret_cast<Vec8<T>*>(out + r * ld_out + c) = o;
  }
}

// ---------------------------------------------------------------- combine
// out[t, :] = sum over j < k of slot_weight[t * k + j] * y[token_rows[t * k + j], :], summed in fp32 in the
// order of j and rounded once.  One workgroup per token; a slot whose row is outside [0, y_rows) adds nothing.
template <typename T>
__global__ void __launch_bounds__(256) moe_combine_kernel(const T* __restrict__ y, const int32_t* __restrict__ token_rows,
                                                          const float* __restrict__ slot_weight, T* __restrict__ out, int k,
                                                          int64_t H, int64_t y_rows, int64_t ld_y, int64_t ld_out) {
  __shared__ int32_t rows[kMaxTopK];
  __shared__ float wts[kMaxTopK];
  const int64_t t = blockIdx.x;
  if (threadIdx.x < k) {
    rows[threadIdx.x] = token_rows[t * k + threadIdx.x];
    wts[threadIdx.x] = slot_weight[t * k + threadIdx.x];
  }
  __syncthreads();
  for (int64_t c = int64_t(threadIdx.x) << 3; c < H; c += 256 * 8) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int j = 0; j < k; ++j) {
      const int64_t r = rows[j];
      if (r < 0 || r >= y_rows) continue;
      const Vec8<T> v = *reinterpret_cast<const Vec8<T>*>(y + r * ld_y + c);
      const float w = wts[j];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] += w * to_float(v.v[i]);
    }
    Vec8<T> o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o.v[i] = from_float<T>(acc[i]);
    *reinterpret_cast<Vec8<T>*>(out + t * ld_out + c) = o;
  }
}

// ---------------------------------------------------------------- host side
bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

struct SortPlan {
  int slots, nb, spb;
};

bool plan_sort(int64_t tokens, int64_t top_k, SortPlan& pl) {
  const int64_t slots = tokens * top_k;
  if (slots < 0 || slots >= (int64_t(1) << 31)) return false;
  int64_t nb = (slots + kSlotsPerSortBlock - 1) / kSlotsPerSortBlock;
  if (nb < 1) nb = 1;
  if (nb > kMaxSortBlocks) nb = kMaxSortBlocks;
  const int64_t spb = slots ? (slots + nb - 1) / nb : 1;
  pl.slots = int(slots);
  pl.spb = int(spb);
  pl.nb = slots ? int((slots + spb - 1) / spb) : 0;
  return true;
}

int route_checked(const void* logits, int64_t ld, int dtype, int64_t tokens, int64_t E, int64_t top_k, int renorm,
                  int32_t* offs, int32_t* slot_expert, float* slot_weight, int32_t* row_token, int32_t* token_rows,
                  int32_t* table, size_t table_bytes, hipStream_t stream) {
  if (tokens < 0 || E < 1 || E > kMaxExperts || top_k < 1 || top_k > kMaxTopK || top_k > E) return GMM_ERR_BAD_ARGUMENT;
  if (dtype < GMM_DT_BF16 || dtype > GMM_DT_F32) return GMM_ERR_UNSUPPORTED;
  SortPlan pl;
  if (!plan_sort(tokens, top_k, pl)) return GMM_ERR_BAD_ARGUMENT;
  if (!offs) return GMM_ERR_BAD_ARGUMENT;
  if (tokens > 0 && (!logits || !slot_expert || !slot_weight || !row_token || !token_rows || ld < E)) return GMM_ERR_BAD_ARGUMENT;
  if (size_t(pl.nb) * size_t(E) * sizeof(int32_t) > table_bytes) return GMM_ERR_WORKSPACE;
  if (pl.nb > 0 && !table) return GMM_ERR_BAD_ARGUMENT;
  if (tokens > 0) {
    const dim3 grid(unsigned((tokens + 3) / 4)), block(256);
    if (dtype == GMM_DT_BF16)
      hipLaunchKernelGGL(moe_topk_kernel<Bf16>, grid, block, 0, stream, static_cast<const Bf16*>(logits), ld, int(tokens), int(E),
                         int(top_k), renorm, slot_expert, slot_weight);
    else if (dtype == GMM_DT_F16)
      hipLaunchKernelGGL(moe_topk_kernel<F16>, grid, block, 0, stream, static_cast<const F16*>(logits), ld, int(tokens), int(E),
                         int(top_k), renorm, slot_expert, slot_weight);
    else
      hipLaunchKernelGGL(moe_topk_kernel<float>, grid, block, 0, stream, static_cast<const float*>(logits), ld, int(tokens), int(E),
                         int(top_k), renorm, slot_expert, slot_weight);
    hipLaunchKernelGGL(moe_hist_kernel, dim3(pl.nb), dim3(256), 0, stream, slot_expert, pl.slots, pl.spb, int(E), table);
  }
  hipLaunchKernelGGL(moe_scan_kernel, dim3(1), dim3(1024), 0, stream, table, pl.nb, int(E), offs);
  if (tokens > 0)
    hipLaunchKernelGGL(moe_scatter_kernel, dim3(pl.nb), dim3(64), 0, stream, slot_expert, pl.slots, pl.spb, int(E), int(top_k),
                       table, offs, row_token, token_rows);
  return hipGetLastError() == hipSuccess ? GMM_OK : GMM_ERR_LAUNCH;
}

// Address of the current device's copy of `scratch`, looked up on the first call on that device.
int32_t* device_scratch() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  int32_t* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    void* sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)) != hipSuccess || !sym) return nullptr;
    p = static_cast<int32_t*>(sym);
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  return p;
}

}  // namespace

extern "C" {

int64_t gmm_moe_route_workspace_bytes(int64_t tokens, int64_t experts, int64_t top_k) {
  SortPlan pl;
  if (tokens < 0 || experts < 1 || experts > kMaxExperts || top_k < 1 || !plan_sort(tokens, top_k, pl)) return -1;
  return int64_t(pl.nb) * experts * int64_t(sizeof(int32_t));
}

int gmm_moe_route(const void* logits, int64_t logits_stride, int32_t logits_dtype, int64_t tokens, int64_t experts,
                  int64_t top_k, int32_t renormalize, int32_t* offs, int32_t* slot_expert, float* slot_weight,
                  int32_t* row_token, int32_t* token_rows, void* workspace, int64_t workspace_bytes, void* stream) {
  if (workspace_bytes < 0) return GMM_ERR_BAD_ARGUMENT;
  return route_checked(logits, logits_stride, logits_dtype, tokens, experts, top_k, renormalize, offs, slot_expert,
                       slot_weight, row_token, token_rows, static_cast<int32_t*>(workspace), size_t(workspace_bytes),
                       static_cast<hipStream_t>(stream));
}

int gmm_moe_route_noalloc(const void* logits, int64_t logits_stride, int32_t logits_dtype, int64_t tokens, int64_t experts,
                          int64_t top_k, int32_t renormalize, int32_t* offs, int32_t* slot_expert, float* slot_weight,
                          int32_t* row_token, int32_t* token_rows, void* stream) {
  int32_t* table = device_scratch();
  if (!table) return GMM_ERR_LAUNCH;
  return route_checked(logits, logits_stride, logits_dtype, tokens, experts, top_k, renormalize, offs, slot_expert,
                       slot_weight, row_token, token_rows, table, sizeof(int32_t) * size_t(kScratchInts),
                       static_cast<hipStream_t>(stream));
}

int gmm_moe_activation(const void* h, void* out, int64_t rows, int64_t inner, int64_t h_stride, int64_t out_stride,
                       int32_t kind, int32_t dtype, void* stream) {
  if (rows < 0 || inner < 0 || kind < 0 || kind > 1) return GMM_ERR_BAD_ARGUMENT;
  if (dtype != GMM_DT_BF16 && dtype != GMM_DT_F16) return GMM_ERR_UNSUPPORTED;
  if (rows == 0 || inner == 0) return GMM_OK;
  if (!h || !out || (inner & 7) || (h_stride & 7) || (out_stride & 7) || !aligned16(h) || !aligned16(out)) return GMM_ERR_BAD_ARGUMENT;
  if (h_stride < (kind ? 2 : 1) * inner || out_stride < inner) return GMM_ERR_BAD_ARGUMENT;
  const int64_t vecs = rows * (inner >> 3);
  int64_t blocks = (vecs + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  const dim3 grid{unsigned(blocks)}, block{256};
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == GMM_DT_BF16)
    hipLaunchKernelGGL(moe_act_kernel<Bf16>, grid, block, 0, s, static_cast<const Bf16*>(h), static_cast<Bf16*>(out), rows, inner,
                       h_stride, out_stride, kind);
  else
    hipLaunchKernelGGL(moe_act_kernel<F16>, grid, block, 0, s, static_cast<const F16*>(h), static_cast<F16*>(out), rows, inner,
                       h_stride, out_stride, kind);
  return hipGetLastError() == hipSuccess ? GMM_OK : GMM_ERR_LAUNCH;
}

int gmm_moe_combine(const void* y, const int32_t* token_rows, const float* slot_weight, void* out, int64_t tokens,
                    int64_t top_k, int64_t hidden, int64_t y_rows, int64_t y_stride, int64_t out_stride, int32_t dtype,
                    void* stream) {
  if (tokens < 0 || tokens >= (int64_t(1) << 31) || top_k < 1 || top_k > kMaxTopK || hidden < 0 || y_rows < 0) return GMM_ERR_BAD_ARGUMENT;
  if (dtype != GMM_DT_BF16 && dtype != GMM_DT_F16) return GMM_ERR_UNSUPPORTED;
  if (tokens == 0 || hidden == 0) return GMM_OK;
  if (!out || !token_rows || !slot_weight || (y_rows > 0 && !y)) return GMM_ERR_BAD_ARGUMENT;
  if ((hidden & 7) || (y_stride & 7) || (out_stride & 7) || !aligned16(y) || !aligned16(out)) return GMM_ERR_BAD_ARGUMENT;
  if (y_stride < hidden || out_stride < hidden) return GMM_ERR_BAD_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid{unsigned(tokens)}, block{256};
  if (dtype == GMM_DT_BF16)
    hipLaunchKernelGGL(moe_combine_kernel<Bf16>, grid, block, 0, s, static_cast<const Bf16*>(y), token_rows, slot_weight,
                       static_cast<Bf16*>(out), int(top_k), hidden, y_rows, y_stride, out_stride);
  else
    hipLaunchKernelGGL(moe_combine_kernel<F16>, grid, block, 0, s, static_cast<const F16*>(y), token_rows, slot_weight,
                       static_cast<F16*>(out), int(top_k), hidden, y_rows, y_stride, out_stride);
  return hipGetLastError() == hipSuccess ? GMM_OK : GMM_ERR_LAUNCH;
}

}  // extern "C"
