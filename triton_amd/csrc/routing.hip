// Top-k softmax router, expert histogram / gather-scatter indices and ragged block schedule for gfx950.
//
// The reference spends six dependent launches here (top-k, vertical popcount, two metadata stages,
// two ragged-metadata kernels).  Here the work is three launches, all latency-bound integer work:
//
//   route_topk_kernel    one wave64 owns a run of `rows_per_wave` tokens.  A row's logits sit in
//                        registers (lane l holds experts l, l+64, ...); each of the k rounds is a
//                        wave-wide max-reduction of a 64-bit key (order-preserving float key in the high
//                        word, ~expert in the low word, so ties go to the LOWER expert id).  The wave
//                        also accumulates its private per-expert histogram in LDS and writes it out
//                        as one row of `partials`.
//   route_scan_kernel    ONE workgroup: per expert an exclusive prefix over the workgroups' histogram totals
//                        (route_topk_kernel sums its four waves' histograms; the scatter adds the earlier waves
//                        of its own workgroup back),
//                        the expert totals (`col_sum`), their exclusive scan (`col_offs`) and, if
//                        asked, the whole ragged metadata (slice offsets, block offsets and block
//                        schedules for block sizes 16..256).
//   route_scatter_kernel each wave re-reads its tokens' expert ids in flat (token-major) order, ranks
//                        equal ids with ballots (stable), and writes both permutations plus the
//                        optional gather index / gate value in expert-sorted order.
#include <mutex>

#include "common.h"
#include "route_common.h"

namespace tk {
namespace {

constexpr int kMaxExperts = 2048;  // per-wave LDS histogram: 4 waves x 2048 x 4 B = 32 KiB
constexpr int kWaves = 4;
constexpr int kNumBlockSizes = 5;  // 16, 32, 64, 128, 256
constexpr int kFirstBlockLog2 = 4;

template <int DT>
__device__ inline float load_logit(const void* p, int64_t i) {
  if (DT == TK_F32) return static_cast<const float*>(p)[i];
  if (DT == TK_BF16) return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
  return f16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
}
template <int DT>
__device__ inline void store_val(void* p, int64_t i, float v) {
  if (DT == TK_F32)
    static_cast<float*>(p)[i] = v;
  else if (DT == TK_BF16)
    static_cast<uint16_t*>(p)[i] = f32_to_bf16_bits(v);
  else
    static_cast<uint16_t*>(p)[i] = f32_to_f16_bits(v);
}

struct TopkParams {
  const void* logits;  // [T, E] or null (histogram of given indices only)
  int64_t stride_m;
  int32_t T;
  int32_t n_rows_imm;
  const int32_t* n_rows_ptr;
  int32_t E, k;
  int32_t apply_softmax;
  int32_t use_provided_indx;
  void* vals;               // [T, k] logits dtype, or null
  int16_t* indx;            // [T, k]
  uint32_t* bitmatrix;      // [words][T_pad] or null
  int64_t bm_stride_w;
  int32_t* partials;        // [units][E] or null
  int32_t* wg_totals;       // [workgroups][E] (with partials): the histograms of a workgroup's waves summed
  int32_t rows_per_wave;
  int32_t* fill_a;          // [T*k] arrays preset to -1 (the two permutations and the gather index), or null
  int32_t* fill_b;
  int32_t* fill_c;
};

// PROVIDED = the caller supplies the expert indices (p.use_provided_indx); as a template parameter so that the selecting
// variant has no load inside its row loop: with one on some path the compiler waits for ALL outstanding memory
// operations at the joins, i.e. for the previous row's stores.
template <int DT, int EPL, bool PROVIDED>
__global__ __launch_bounds__(kWaves * 64) void route_topk_kernel(const TopkParams p) {
  __shared__ int32_t hist_s[kWaves][EPL * 64];
  __shared__ uint32_t words_s[kWaves][EPL * 2];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int unit = blockIdx.x * kWaves + wave;
  const int E = p.E, k = p.k;
  const int n_rows = p.n_rows_ptr ? *p.n_rows_ptr : p.n_rows_imm;
  const int words = (E + 31) / 32;
  for (int e = lane; e < EPL * 64; e += 64) hist_s[wave][e] = 0;
  const int row_begin = unit * p.rows_per_wave;
  int row_end = row_begin + p.rows_per_wave;
  row_end = row_end < p.T ? row_end : p.T;
  if (p.fill_a) {
    // entries that are never routed (masked rows, dropped indices) leave -1 in the permutations
    for (int64_t f = (int64_t)row_begin * k + lane; f < (int64_t)row_end * k; f += 64) {
      p.fill_a[f] = -1;
      p.fill_b[f] = -1;
      if (p.fill_c) p.fill_c[f] = -1;
    }
  }
  // The logits of up to kBatch rows are fetched together before the first of them is selected: a wave walks its rows
  // one after the other, and with one row in flight at a time every row cost a full memory latency.
  constexpr int kBatch = EPL <= 2 ? 8 : EPL <= 4 ? 4 : EPL <= 8 ? 2 : 1;
  float batch_v[kBatch][EPL];
  for (int row0 = row_begin; row0 < row_end; row0 += kBatch) {
  if constexpr (!PROVIDED) {
#pragma unroll
    for (int r = 0; r < kBatch; ++r) {
      const int row = row0 + r;
      // (no conditions around the loads: rows past the run repeat its last row and are never used, columns past E the
      // last column and their keys are retired; behind a condition every load of a 16-bit row got a wait of its own)
      const int64_t at = (int64_t)(row < row_end ? row : row_end - 1) * p.stride_m;
#pragma unroll
      for (int i = 0; i < EPL; ++i) {
        const int e = lane + 64 * i;
        batch_v[r][i] = load_logit<DT>(p.logits, at + (e < E ? e : E - 1));
      }
    }
  }
  // The keys of the whole batch are taken HERE, in front of the first row's stores.  Loads and stores of a wave complete
  // in order and share one counter, the stores below sit behind conditions, so the compiler counts none of them: a wait
  // for a later row's logits placed behind an earlier row's stores waits for those stores as well, a memory round trip
  // per row.
  uint32_t bkey[kBatch][EPL];
  if constexpr (!PROVIDED) {
#pragma unroll
    for (int r = 0; r < kBatch; ++r)
#pragma unroll
      for (int i = 0; i < EPL; ++i) {
        bkey[r][i] = lane + 64 * i < E ? ordered_key(batch_v[r][i]) : 0u;
        asm volatile("" ::"v"(bkey[r][i]) : "memory");
      }
  }
#pragma unroll
  for (int r = 0; r < kBatch; ++r) {
    const int row = row0 + r;
    if (row >= row_end || row >= n_rows) break;
    float myval = 0.f;
    int myidx = -1;
    if constexpr (PROVIDED) {
      if (lane < k) {
        myidx = p.indx[(int64_t)row * k + lane];
        if (p.logits && myidx >= 0) myval = load_logit<DT>(p.logits, (int64_t)row * p.stride_m + myidx);
      }
    } else {
      wave_topk<EPL>(bkey[r], k, E, lane, myval, myidx);
    }
    float outv = myval;
    if (p.apply_softmax) {
      // softmax over the k kept logits in fp32; the largest sits in lane 0
      float vmax = myval;
      if constexpr (PROVIDED) {
        float m = lane < k ? myval : -INFINITY;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
        vmax = m;
      } else {
        vmax = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, myval), 0));
      }
      const float z = lane < k ? expf(myval - vmax) : 0.f;
      const float sum = wave_sum_f32(z);
      outv = z / sum;
    }
    if (lane < k) {
      if (p.vals) store_val<DT>(p.vals, (int64_t)row * k + lane, outv);
      if constexpr (!PROVIDED) p.indx[(int64_t)row * k + lane] = (int16_t)myidx;
    }
    const bool live = lane < k && myidx >= 0 && myidx < E;
    if (p.partials && live) atomicAdd(&hist_s[wave][myidx], 1);
    if (p.bitmatrix) {
      // (words <= 64: at most 2048 experts.  No loops here: the compiler drains all outstanding global stores in front
      // of a loop that touches memory, which would cost every row a store latency.)
      if (lane < words) words_s[wave][lane] = 0u;
      wave_sync();
      if (live) atomicOr(&words_s[wave][myidx >> 5], 1u << (myidx & 31));
      wave_sync();
      if (lane < words) p.bitmatrix[(int64_t)lane * p.bm_stride_w + row] = words_s[wave][lane];
      wave_sync();
    }
  }
  }
  if (p.partials) {
    if (row_begin < p.T) {
      wave_sync();
      for (int e = lane; e < E; e += 64) p.partials[(int64_t)unit * E + e] = hist_s[wave][e];
    }
    // the workgroup's total per expert: the scan walks these rows, a quarter as many as there are waves
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += kWaves * 64) {
      int t = 0;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) t += hist_s[w][e];
      p.wg_totals[(int64_t)blockIdx.x * E + e] = t;
    }
  }
}

// ---- block-wide exclusive scan (1024 threads) ---------------------------------------------------
constexpr int kScanThreads = 1024;

struct RaggedOut {
  int32_t* slice_offs;    // [E+1] or null
  int32_t* block_offs;    // [kNumBlockSizes][stride] or null
  int64_t block_offs_stride;
  int32_t* block_sched;   // [kNumBlockSizes][stride]
  int64_t block_sched_stride;
  int32_t max_n_blocks;
};

constexpr int kScanWaves = kScanThreads / 64;
constexpr int kQuantities = 1 + kNumBlockSizes;  // rows, then row blocks of 16, 32, 64, 128, 256

// Exclusive scans of the slice sizes and of their block counts for all block sizes in ONE pass over the
// slices: each thread carries the six quantities of its slice through a wave scan, the wave totals are
// exchanged once through LDS.  offs0 (optional) and r.slice_offs (optional) receive the row offsets,
// r.block_offs the block offsets.  Then every schedule slot finds its slice by binary search in the
// block offsets, so a slice with thousands of blocks costs no more than an empty one.
constexpr int kLdsOffsExperts = 1024;  // up to this many slices the offsets are also kept in LDS

// Returns the LDS copy of the slice offsets ([E + 1], valid after the caller's next workgroup barrier) or null when E
// is too large for it.
__device__ __forceinline__ const int32_t* ragged_metadata(const int32_t* slice_sizes, int E, int32_t* offs0, const RaggedOut r, bool want_ragged) {
  // LDS copies: row 0 = slice offsets (read back by the single-launch router), rows 1.. = block offsets, which the
  // schedule's binary search reads (seven dependent reads per slot; from global memory they dominated the kernel)
  __shared__ int32_t offs_s[kQuantities][kLdsOffsExperts + 1];
  const bool use_lds = E <= kLdsOffsExperts;
  __shared__ int wave_tot[kQuantities][kScanWaves + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nq = want_ragged ? kQuantities : 1;
  int carry[kQuantities];
#pragma unroll
  for (int q = 0; q < kQuantities; ++q) carry[q] = 0;
  for (int base = 0; base < E; base += kScanThreads) {
    const int i = base + threadIdx.x;
    const int sz = i < E ? slice_sizes[i] : 0;
    int v[kQuantities], inc[kQuantities];
    v[0] = sz;
#pragma unroll
    for (int b = 0; b < kNumBlockSizes; ++b) v[1 + b] = (sz + ((1 << (kFirstBlockLog2 + b)) - 1)) >> (kFirstBlockLog2 + b);
#pragma unroll
    for (int q = 0; q < kQuantities; ++q) inc[q] = wave_scan_i32(v[q]);  // (DPP: six lane exchanges through LDS each took 2 us more)
    __syncthreads();  // wave_tot may still be read by the previous trip
    if (lane == 63) {
#pragma unroll
      for (int q = 0; q < kQuantities; ++q) wave_tot[q][wave] = inc[q];
    }
    __syncthreads();
    if (threadIdx.x < kQuantities) {
      // (only the waves that hold slices of this trip: with 128 experts two of the sixteen, and every step of this walk
      // is an LDS round trip)
      const int left = E - base;
      const int used = left >= kScanThreads ? kScanWaves : (left + 63) >> 6;
      int run = 0;
      for (int w = 0; w < used; ++w) {
        const int t = wave_tot[threadIdx.x][w];
        wave_tot[threadIdx.x][w] = run;
        run += t;
      }
      for (int w = used; w < kScanWaves; ++w) wave_tot[threadIdx.x][w] = run;
      wave_tot[threadIdx.x][kScanWaves] = run;
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < kQuantities; ++q) {
      if (q < nq && i < E) {
        const int ex = carry[q] + wave_tot[q][wave] + inc[q] - v[q];
        if (use_lds) offs_s[q][i] = ex;
        if (q == 0) {
          if (offs0) offs0[i] = ex;
          if (want_ragged) r.slice_offs[i] = ex;
        } else {
          r.block_offs[(q - 1) * r.block_offs_stride + i] = ex;
        }
      }
      carry[q] += wave_tot[q][kScanWaves];
    }
  }
  if (threadIdx.x == 0) {
    if (offs0) offs0[E] = carry[0];
    if (use_lds) {
#pragma unroll
      for (int q = 0; q < kQuantities; ++q) offs_s[q][E] = carry[q];
    }
    if (want_ragged) {
      r.slice_offs[E] = carry[0];
#pragma unroll
      for (int b = 0; b < kNumBlockSizes; ++b) r.block_offs[b * r.block_offs_stride + E] = carry[1 + b];
    }
  }
  if (!want_ragged) return use_lds ? offs_s[0] : nullptr;
  __threadfence_block();
  __syncthreads();
  // (the slots of all block sizes in ONE loop: with a few hundred slots per size the five searches of a thread, seven
  // dependent LDS reads each, run side by side in different threads instead of one after the other)
  const int n_slots = kNumBlockSizes * r.max_n_blocks;
  for (int slot = threadIdx.x; slot < n_slots; slot += kScanThreads) {
    const int b = slot / r.max_n_blocks, i = slot - b * r.max_n_blocks;
    const int32_t* offs = use_lds ? offs_s[1 + b] : r.block_offs + b * r.block_offs_stride;
    int tot = 0;  // blocks of this size in all slices (every thread has carried the totals through the scan)
#pragma unroll
    for (int bb = 0; bb < kNumBlockSizes; ++bb) tot = bb == b ? carry[1 + bb] : tot;
    int val = -1;
    if (i < tot) {
      int lo = 0, hi = E;  // largest e with offs[e] <= i; empty slices share an offset, the last one wins
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (offs[mid] <= i) lo = mid; else hi = mid;
      }
      val = ((i - offs[lo]) << 16) | lo;
    }
    r.block_sched[b * r.block_sched_stride + i] = val;
  }
  return use_lds ? offs_s[0] : nullptr;
}

// Exclusive prefix over the waves' histograms, per expert.  Threads are laid out [group][expert] so that a
// wave reads consecutive experts of one unit (coalesced); the units are split into `groups` contiguous
// runs that are summed in parallel (pass 1), offset by an LDS exchange of the run totals, and rewritten
// as exclusive prefixes (pass 2) with the loads of a chunk issued before its dependent stores.
__global__ __launch_bounds__(kScanThreads) void route_scan_kernel(int32_t* partials, int units, int E, int32_t* col_sum,
                                                                  int32_t* col_offs, int want_ragged, const RaggedOut r) {
  __shared__ int32_t run_total[kScanThreads];
  int groups = kScanThreads / E;
  groups = groups < 1 ? 1 : (groups > 32 ? 32 : groups);
  groups = groups > units ? units : groups;
  const int per_group = (units + groups - 1) / groups;
  // loads of a chunk are in flight together: the kernel is one workgroup walking `units` rows of the workspace, and its
  // time is the number of dependent memory round trips (two passes x run length / kChunk)
  constexpr int kChunk = 16;
  // Vector form (E a multiple of 4, the usual case): a thread owns FOUR experts of a run of units and moves them as one
  // 16-byte piece, so 1024 threads cover E / 4 columns x up to 32 runs; a run of at most kVec units stays in registers
  // between the two passes (one memory round trip to read, one to write), longer runs are walked in chunks of kVec.
  constexpr int kVec = 12;
  if (E % 4 == 0 && E / 4 <= kScanThreads && (reinterpret_cast<uintptr_t>(partials) & 15) == 0 && (reinterpret_cast<uintptr_t>(col_sum) & 15) == 0) {
    __shared__ int4 run_total4[kScanThreads];
    const int w4 = E / 4;
    int vgroups = kScanThreads / w4;
    vgroups = vgroups > 32 ? 32 : vgroups;
    vgroups = vgroups > units ? units : vgroups;
    vgroups = vgroups < 1 ? 1 : vgroups;
    const int vper = (units + vgroups - 1) / vgroups;
    const int e4 = (int)(threadIdx.x % (unsigned)w4), g = (int)(threadIdx.x / (unsigned)w4);
    const bool active = g < vgroups;
    const int u_begin = g * vper;
    int u_end = u_begin + vper;
    u_end = u_end < units ? u_end : units;
    int4* p4 = reinterpret_cast<int4*>(partials);
    const bool single = vper <= kVec;
    int4 v[kVec];
    int4 sum = make_int4(0, 0, 0, 0);
    if (active) {
      for (int u = u_begin; u < u_end; u += kVec) {
#pragma unroll
        for (int i = 0; i < kVec; ++i) v[i] = u + i < u_end ? p4[(int64_t)(u + i) * w4 + e4] : make_int4(0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < kVec; ++i) {
          sum.x += v[i].x;
          sum.y += v[i].y;
          sum.z += v[i].z;
          sum.w += v[i].w;
        }
      }
      run_total4[threadIdx.x] = sum;
    }
    __syncthreads();
    if (active) {
      int4 run = make_int4(0, 0, 0, 0);
      for (int gg = 0; gg < g; ++gg) {
        const int4 t = run_total4[gg * w4 + e4];
        run.x += t.x;
        run.y += t.y;
        run.z += t.z;
        run.w += t.w;
      }
      for (int u = u_begin; u < u_end; u += kVec) {
        if (!single) {
#pragma unroll
          for (int i = 0; i < kVec; ++i) v[i] = u + i < u_end ? p4[(int64_t)(u + i) * w4 + e4] : make_int4(0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < kVec; ++i) {
          if (u + i < u_end) p4[(int64_t)(u + i) * w4 + e4] = run;
          run.x += v[i].x;
          run.y += v[i].y;
          run.z += v[i].z;
          run.w += v[i].w;
        }
      }
      if (g == vgroups - 1) reinterpret_cast<int4*>(col_sum)[e4] = run;
    }
  } else
  for (int e0 = 0; e0 < E; e0 += kScanThreads) {  // more than one trip only when E > 1024 (then groups == 1)
    const int e = e0 + (int)(threadIdx.x % (unsigned)(E < kScanThreads ? E : kScanThreads));
    const int g = (int)(threadIdx.x / (unsigned)(E < kScanThreads ? E : kScanThreads));
    const bool active = e < E && g < groups;
    const int u_begin = g * per_group;
    int u_end = u_begin + per_group;
    u_end = u_end < units ? u_end : units;
    int sum = 0;
    if (active) {
      int u = u_begin;
      for (; u + kChunk <= u_end; u += kChunk) {
        int v[kChunk];
#pragma unroll
        for (int i = 0; i < kChunk; ++i) v[i] = partials[(int64_t)(u + i) * E + e];
#pragma unroll
        for (int i = 0; i < kChunk; ++i) sum += v[i];
      }
      for (; u < u_end; ++u) sum += partials[(int64_t)u * E + e];
    }
    __syncthreads();  // run_total may still be read by the previous trip
    if (active) run_total[threadIdx.x] = sum;
    __syncthreads();
    if (active) {
      const int width = E < kScanThreads ? E : kScanThreads;
      int run = 0;
      for (int gg = 0; gg < g; ++gg) run += run_total[gg * width + (e - e0)];
      int u = u_begin;
      for (; u + kChunk <= u_end; u += kChunk) {
        int v[kChunk];
#pragma unroll
        for (int i = 0; i < kChunk; ++i) v[i] = partials[(int64_t)(u + i) * E + e];
#pragma unroll
        for (int i = 0; i < kChunk; ++i) {
          partials[(int64_t)(u + i) * E + e] = run;
          run += v[i];
        }
      }
      for (; u < u_end; ++u) {
        const int t = partials[(int64_t)u * E + e];
        partials[(int64_t)u * E + e] = run;
        run += t;
      }
      if (g == groups - 1) col_sum[e] = run;
    }
  }
  __threadfence_block();
  __syncthreads();
  ragged_metadata(col_sum, E, col_offs, r, want_ragged != 0);
}

__global__ __launch_bounds__(kScanThreads) void ragged_metadata_kernel(const int32_t* slice_sizes, int E, const RaggedOut r) {
  ragged_metadata(slice_sizes, E, nullptr, r, true);
}

// ---- top-k backward ---------------------------------------------------------------------------------------
// dx[row, :] = 0 except dx[row, indx[row, j]] = y_j * (dy_j - sum_i y_i dy_i) with y = softmax of the k kept logits
// (recomputed in fp32), or dy_j without softmax (topk_details/_topk_backward.py:5-51 of the reference).  One wave per
// row; every dx element is written once, by the lane that owns its column.
template <int DT>
__global__ __launch_bounds__(256) void topk_backward_kernel(const void* x, int64_t stride_xm, const int16_t* indx, int64_t stride_im,
                                                            const void* dy, int64_t stride_dym, void* dx, int64_t stride_dxm, int T,
                                                            int E, int k, int apply_softmax, int n_rows_imm, const int32_t* n_rows_ptr) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= T) return;
  const int n_rows = n_rows_ptr ? *n_rows_ptr : n_rows_imm;
  int idx = -1;
  float g = 0.f;
  if (row < n_rows) {
    float xv = -INFINITY, dyv = 0.f;
    if (lane < k) {
      idx = indx[(int64_t)row * stride_im + lane];
      if (idx < 0 || idx >= E) idx = -1;
      if (idx >= 0) {
        xv = load_logit<DT>(x, (int64_t)row * stride_xm + idx);
        dyv = load_logit<DT>(dy, (int64_t)row * stride_dym + lane);
      }
    }
    g = dyv;
    if (apply_softmax) {
      float m = xv;
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
      const float z = idx >= 0 ? expf(xv - m) : 0.f;
      const float sum = wave_sum_f32(z);
      const float y = sum > 0.f ? z / sum : 0.f;
      const float s = wave_sum_f32(y * dyv);
      g = y * (dyv - s);
    }
  }
  for (int e0 = 0; e0 < E; e0 += 64) {
    const int e = e0 + lane;
    float out = 0.f;
    for (int j = 0; j < k; ++j) {
      const int ij = __shfl(idx, j);
      const float gj = __shfl(g, j);
      out = (ij == e) ? gj : out;
    }
    if (e < E) store_val<DT>(dx, (int64_t)row * stride_dxm + e, out);
  }
}

// ---- remapping ragged metadata to a subset of the slices ------------------------------------------------
// Order-preserving compaction by a 1024-thread workgroup: out[rank(i)] = value(i) for the kept i, -1 behind them.
// `f(i, v)` yields element i's value and whether it is kept.  Returns the number kept (uniform).
template <class F>
__device__ __forceinline__ int compact_block(int32_t* out, int n, int* wave_tot, F&& f) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int base = 0;
  for (int start = 0; start < n; start += kScanThreads) {
    const int i = start + threadIdx.x;
    int32_t v = -1;
    const bool keep = i < n && f(i, v);
    const unsigned long long mask = __ballot(keep);
    if (lane == 0) wave_tot[wave] = __builtin_popcountll(mask);
    __syncthreads();
    int before = 0, total = 0;
    for (int w = 0; w < kScanThreads / 64; ++w) {
      const int t = wave_tot[w];
      before += w < wave ? t : 0;
      total += t;
    }
    if (keep) out[base + before + __builtin_popcountll(mask & ((1ull << lane) - 1ull))] = v;
    base += total;
    __syncthreads();
  }
  for (int i = base + threadIdx.x; i < n; i += kScanThreads) out[i] = -1;
  return base;
}

struct RemapParams {
  const int32_t* slice_sizes;
  const int32_t* slice_offs;
  const int32_t* block_offs;
  int64_t block_offs_stride;
  const int32_t* block_sched;
  int64_t block_sched_stride;
  const int32_t* slice_map;
  int32_t n_slices, max_n_blocks;
  int32_t* slice_sizes_out;
  int32_t* slice_offs_out;
  int32_t* block_offs_out;
  int64_t block_offs_out_stride;
  int32_t* block_sched_out;
  int64_t block_sched_out_stride;
};

// Workgroup 0 compacts the slice sizes and offsets; workgroup 1 + b the block offsets and the block schedule of
// block size b, whose entries get the slice's new id; the count of the schedule entries kept goes behind the kept
// block offsets (tensor_details/ragged_tensor.py:309-345 of the reference).
__global__ __launch_bounds__(kScanThreads) void ragged_remap_kernel(const RemapParams p) {
  __shared__ int wave_tot[kScanThreads / 64];
  const int n = p.n_slices;
  const int32_t* map = p.slice_map;
  auto kept_slice = [&](int i) { return i < n && map[i] != -1; };
  if (blockIdx.x == 0) {
    compact_block(p.slice_sizes_out, n, wave_tot, [&](int i, int32_t& v) { v = p.slice_sizes[i]; return kept_slice(i); });
    compact_block(p.slice_offs_out, n + 1, wave_tot, [&](int i, int32_t& v) { v = p.slice_offs[i]; return kept_slice(i); });
    return;
  }
  const int b = blockIdx.x - 1;
  const int32_t* bo = p.block_offs + b * p.block_offs_stride;
  const int32_t* bs = p.block_sched + b * p.block_sched_stride;
  int32_t* bo_out = p.block_offs_out + b * p.block_offs_out_stride;
  const int n_kept = compact_block(bo_out, n + 1, wave_tot, [&](int i, int32_t& v) { v = bo[i]; return kept_slice(i); });
  const int n_blocks = compact_block(p.block_sched_out + b * p.block_sched_out_stride, p.max_n_blocks, wave_tot, [&](int i, int32_t& v) {
    const uint32_t e = (uint32_t)bs[i];
    const uint32_t slice = e & 0xFFFFu;
    if (slice == 0xFFFFu || (int)slice >= n) return false;  // unused tail of the schedule
    const int32_t to = map[slice];
    v = (int32_t)((e & 0xFFFF0000u) | ((uint32_t)to & 0xFFFFu));
    return to != -1;
  });
  __syncthreads();
  if (threadIdx.x == 0) bo_out[n_kept] = n_blocks;
}

// ---- whole routing pass in ONE workgroup (small batches) ------------------------------------------
// For T*k <= kSmallEntries the three phases run back to back in a single 1024-thread workgroup: the waves take
// rows round-robin for the top-k, the selected expert ids stay in LDS, the histogram is built with LDS atomics,
// an entry's stable rank inside its expert is a count over the earlier entries (at most kSmallEntries LDS
// reads, all lanes reading the same address), and the ragged metadata follows.  One launch instead of three:
// at decode batch sizes the pass is pure launch latency.
constexpr int kSmallEntries = 1024;
// ... and is USED up to this many entries: the single workgroup is bound by one CU's instruction rate (sixteen waves share
// four SIMDs), so its top-k phase grows with the batch (inside the launch 6.6 us at 64 entries, 9.9 at 256, 22.7 at 1024)
// while the three kernels, spread over the chip, stay at 20 us from launch to end: at 384 / 512 / 768 / 1024 entries a
// replayed graph measured 24.8 / 27.2 / 34.4 / 42.6 us for the single launch against 19.8 / 20.5 / 19.8 / 20.5.
constexpr int kSmallCut = 256;

struct SmallParams {
  TopkParams t;
  int32_t* col_sum;
  int32_t* col_offs;  // [E+1] scratch
  int32_t* col_sorted;
  int32_t* row_sorted;
  int32_t* gather_out;
  void* gammas_out;
  int32_t vals_bytes;
  int32_t want_ragged;
  RaggedOut r;
};

template <int DT, int EPL, bool PROVIDED>
__global__ __launch_bounds__(kScanThreads) void route_small_kernel(const SmallParams q) {
  __shared__ __attribute__((aligned(16))) int32_t eid_s[kSmallEntries];
  __shared__ uint32_t val_s[kSmallEntries];
  __shared__ int32_t hist_s[kMaxExperts];
  __shared__ uint32_t words_s[kScanWaves][4 * EPL * 2];  // bitmatrix words of the rows a wave has in hand (up to four)
  const TopkParams& p = q.t;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int E = p.E, k = p.k, T = p.T;
  const int n_rows = p.n_rows_ptr ? *p.n_rows_ptr : p.n_rows_imm;
  const int words = (E + 31) / 32;
  const int R = T * k;
  for (int e = threadIdx.x; e < E; e += kScanThreads) hist_s[e] = 0;
  for (int f = threadIdx.x; f < R; f += kScanThreads) eid_s[f] = -1;
  __syncthreads();
  // ---- phase 1: top-k per row (wave w takes rows w, w + 16, ...); the next row's logits are fetched while the
  // current row is selected, so a wave pays the memory latency once ----
  // (rows in batches, all loads of a batch in flight together and none inside the per-row code: see route_topk_kernel)
  constexpr bool kRows4 = !PROVIDED && EPL <= 8;  // (up to 512 experts: a lane holds at most 32 keys)
  // (with more rows than waves only; and k <= 16, where the gate values come out bit for bit as from the row-per-wave
  // code below: the sums meet the same values in the same lanes of a DPP row)
  bool rows4 = false;
  if constexpr (kRows4) rows4 = k <= 16 && T > kScanWaves && n_rows > kScanWaves;
  if constexpr (kRows4) if (rows4) {
    // FOUR rows per wave at a time: the sixteen lanes of a DPP row own a row (row16_topk), so 64 rows are in hand per
    // pass of the sixteen waves instead of 16, and a wave's pass costs what one row cost (about 1.7 us); the next
    // pass's logits are fetched before this pass's rows are selected.
    constexpr int VPL = EPL * 4, W = EPL * 2;
    const int l16 = lane & 15, sub = lane >> 4;
    const int n_live = T < n_rows ? T : n_rows;
    float cur[VPL], nxt[VPL];
    // (loads without conditions: a row past the last repeats the last row, a column past E the last column; their keys
    // are retired or their rows never written.  Behind a condition each load got a branch and a wait of its own.)
    auto fetch = [&](int r, float (&dst)[VPL]) __attribute__((always_inline)) {
      const int64_t at = (int64_t)(r < T ? r : T - 1) * p.stride_m;
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const int e = l16 * VPL + i;
        dst[i] = load_logit<DT>(p.logits, at + (e < E ? e : E - 1));
      }
    };
    fetch(wave * 4 + sub, cur);
    uint32_t key[VPL];
    uint32_t retired = 0;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      key[i] = ordered_key(cur[i]);
      retired |= (l16 * VPL + i >= E ? 1u : 0u) << i;
    }
    for (int row0 = 0; row0 + wave * 4 < n_live; row0 += kScanWaves * 4) {
      const int row = row0 + wave * 4 + sub;
      const bool row_ok = row < n_live;
      fetch(row + kScanWaves * 4, nxt);
      uint32_t sel_key[2] = {0u, 0u};
      int sel_idx[2] = {0x7FFFFFFF, 0x7FFFFFFF};
      uint32_t key0 = 0;
      row16_topk<VPL>(key, retired, k, l16, sel_key, sel_idx, key0);
      float outv[2], z[2];
      const float vmax = key_to_float(key0);
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        outv[h] = key_to_float(sel_key[h]);
        z[h] = l16 + 16 * h < k ? expf(outv[h] - vmax) : 0.f;
      }
      if (p.apply_softmax) {
        const float sum = row16_sum_f32(z[0] + z[1]);
        outv[0] = z[0] / sum;
        outv[1] = z[1] / sum;
      }
      // The next pass's keys are taken HERE, in front of this pass's stores.  Loads and stores of a wave complete in
      // order and share one counter, the stores below sit behind conditions, so the compiler counts none of them: a
      // wait for these loads placed behind the stores would wait for every store as well, a memory round trip per pass.
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        key[i] = ordered_key(nxt[i]);
        asm volatile("" ::"v"(key[i]) : "memory");
      }
      if (p.bitmatrix) {
        if (l16 < words) words_s[wave][sub * W + l16] = 0u;
        wave_sync();
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int j = l16 + 16 * h;
        if (row_ok && j < k) {
          const int myidx = sel_idx[h];
          const bool live = myidx >= 0 && myidx < E;
          if (p.vals) store_val<DT>(p.vals, (int64_t)row * k + j, outv[h]);
          p.indx[(int64_t)row * k + j] = (int16_t)(live ? myidx : -1);
          eid_s[row * k + j] = live ? myidx : -1;
          uint32_t bits;  // the gate value as it is stored (bits of the logits dtype)
          if (DT == TK_F32)
            bits = f32_bits(outv[h]);
          else if (DT == TK_BF16)
            bits = f32_to_bf16_bits(outv[h]);
          else
            bits = f32_to_f16_bits(outv[h]);
          val_s[row * k + j] = bits;
          if (live) {
            atomicAdd(&hist_s[myidx], 1);
            if (p.bitmatrix) atomicOr(&words_s[wave][sub * W + (myidx >> 5)], 1u << (myidx & 31));
          }
        }
      }
      if (p.bitmatrix) {
        wave_sync();
        if (row_ok && l16 < words) p.bitmatrix[(int64_t)l16 * p.bm_stride_w + row] = words_s[wave][sub * W + l16];
        wave_sync();
      }
    }
  }
  if (!rows4) {
  constexpr int kBatch = EPL <= 2 ? 4 : EPL <= 8 ? 2 : 1;
  float nv[kBatch][EPL];
  for (int row0 = wave; row0 < T && row0 < n_rows; row0 += kScanWaves * kBatch) {
  if constexpr (!PROVIDED) {
#pragma unroll
    for (int r = 0; r < kBatch; ++r) {
      const int row = row0 + r * kScanWaves;
      // (no conditions around the loads: rows past the last repeat the last row and are never used, columns past E
      // the last column and their keys are retired; behind a condition every load of a 16-bit row got a wait of its own)
      const int64_t at = (int64_t)(row < T ? row : T - 1) * p.stride_m;
#pragma unroll
      for (int i = 0; i < EPL; ++i) {
        const int e = lane + 64 * i;
        nv[r][i] = load_logit<DT>(p.logits, at + (e < E ? e : E - 1));
      }
    }
  }
  // The keys of the whole batch are taken HERE, in front of the first row's stores.  Loads and stores of a wave complete
  // in order and share one counter, the stores below sit behind conditions, so the compiler counts none of them: a wait
  // for a later row's logits placed behind an earlier row's stores waits for those stores as well, a memory round trip
  // per row.
  uint32_t bkey[kBatch][EPL];
  if constexpr (!PROVIDED) {
#pragma unroll
    for (int r = 0; r < kBatch; ++r)
#pragma unroll
      for (int i = 0; i < EPL; ++i) {
        bkey[r][i] = lane + 64 * i < E ? ordered_key(nv[r][i]) : 0u;
        asm volatile("" ::"v"(bkey[r][i]) : "memory");
      }
  }
#pragma unroll
  for (int r = 0; r < kBatch; ++r) {
    const int row = row0 + r * kScanWaves;
    if (row >= T || row >= n_rows) break;
    float myval = 0.f;
    int myidx = -1;
    if constexpr (PROVIDED) {
      if (lane < k) {
        myidx = p.indx[(int64_t)row * k + lane];
        if (p.logits && myidx >= 0) myval = load_logit<DT>(p.logits, (int64_t)row * p.stride_m + myidx);
      }
    } else {
      wave_topk<EPL>(bkey[r], k, E, lane, myval, myidx);
    }
    float outv = myval;
    if (p.apply_softmax) {
      float vmax;
      if constexpr (PROVIDED) {
        float m = lane < k ? myval : -INFINITY;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
        vmax = m;
      } else {
        vmax = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, myval), 0));
      }
      const float z = lane < k ? expf(myval - vmax) : 0.f;
      const float sum = wave_sum_f32(z);
      outv = z / sum;
    }
    const bool live = lane < k && myidx >= 0 && myidx < E;
    if (lane < k) {
      if (p.vals) store_val<DT>(p.vals, (int64_t)row * k + lane, outv);
      if constexpr (!PROVIDED) p.indx[(int64_t)row * k + lane] = (int16_t)myidx;
      eid_s[row * k + lane] = live ? myidx : -1;
      // the gate value as it is stored (bits of the logits dtype)
      uint32_t bits;
      if (DT == TK_F32)
        bits = f32_bits(outv);
      else if (DT == TK_BF16)
        bits = f32_to_bf16_bits(outv);
      else
        bits = f32_to_f16_bits(outv);
      val_s[row * k + lane] = bits;
    }
    if (live) atomicAdd(&hist_s[myidx], 1);
    if (p.bitmatrix) {
      // (words <= 64: at most 2048 experts.  No loops here: the compiler drains all outstanding global stores in front
      // of a loop that touches memory, which would cost every row a store latency.)
      if (lane < words) words_s[wave][lane] = 0u;
      wave_sync();
      if (live) atomicOr(&words_s[wave][myidx >> 5], 1u << (myidx & 31));
      wave_sync();
      if (lane < words) p.bitmatrix[(int64_t)lane * p.bm_stride_w + row] = words_s[wave][lane];
      wave_sync();
    }
  }
  }
  }
  __syncthreads();
  if (!q.col_sum) return;  // top-k only
  // ---- phase 2: histogram out, offsets and ragged metadata ----
  for (int e = threadIdx.x; e < E; e += kScanThreads) q.col_sum[e] = hist_s[e];
  const int32_t* offs_l = ragged_metadata(hist_s, E, q.col_offs, q.r, q.want_ragged != 0);  // sizes straight from LDS
  __threadfence_block();
  __syncthreads();
  // ---- phase 3: stable ranks and the permutations (the offsets come from the LDS copy when there is one: reading
  // back what this workgroup has just written to global memory costs a full memory round trip) ----
  const int32_t* offs = offs_l ? offs_l : q.col_offs;
  int total = offs[E];
  for (int f = threadIdx.x; f < R; f += kScanThreads) {
    const int e = eid_s[f];
    int pos = -1;
    if (e >= 0) {
      // entries of the same expert in front of this one: four per 16-byte LDS read, the reads independent of one
      // another (one entry per read and trip was a chain of LDS round trips as long as the batch)
      int rank = 0;
      const int f4 = f & ~3;
#pragma unroll 4
      for (int g = 0; g < f4; g += 4) {
        const int4 v = *reinterpret_cast<const int4*>(&eid_s[g]);
        rank += (v.x == e ? 1 : 0) + (v.y == e ? 1 : 0) + (v.z == e ? 1 : 0) + (v.w == e ? 1 : 0);
      }
      for (int g = f4; g < f; ++g) rank += eid_s[g] == e ? 1 : 0;
      pos = offs[e] + rank;
      q.col_sorted[pos] = f;
      if (q.gather_out) q.gather_out[pos] = f / k;
      if (q.gammas_out) {
        if (q.vals_bytes == 4)
          static_cast<uint32_t*>(q.gammas_out)[pos] = val_s[f];
        else
          static_cast<uint16_t*>(q.gammas_out)[pos] = (uint16_t)val_s[f];
      }
    }
    q.row_sorted[f] = pos;
  }
  // positions past the routed entries
  for (int i = total + threadIdx.x; i < R; i += kScanThreads) {
    q.col_sorted[i] = -1;
    if (q.gather_out) q.gather_out[i] = -1;
  }
}

struct ScatterParams {
  const int16_t* indx16;  // [T, k] (one of indx16 / indx32)
  const int32_t* indx32;
  int32_t T, k, E;
  int32_t n_rows_imm;
  const int32_t* n_rows_ptr;
  int32_t rows_per_wave;
  const int32_t* partials;  // [units][E]: every wave's own histogram
  const int32_t* wg_prefix; // [workgroups][E]: entries of the expert in earlier workgroups (exclusive scan of the totals)
  const int32_t* col_offs;  // [E+1]
  int32_t* col_sorted;      // [T*k]
  int32_t* row_sorted;      // [T*k]
  int32_t* gather_out;      // [T*k] or null: token feeding sorted row
  const void* vals;         // [T, k] or null
  void* gammas_out;         // [T*k] or null: gate value of sorted row (same dtype as vals)
  int32_t vals_bytes;       // 2 or 4
};

__global__ __launch_bounds__(kWaves * 64) void route_scatter_kernel(const ScatterParams p) {
  __shared__ int32_t base_s[kWaves][kMaxExperts];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int unit = blockIdx.x * kWaves + wave;
  const int E = p.E, k = p.k;
  const int n_rows = p.n_rows_ptr ? *p.n_rows_ptr : p.n_rows_imm;
  const int row_begin = unit * p.rows_per_wave;
  if (row_begin >= p.T) return;
  int row_end = row_begin + p.rows_per_wave;
  row_end = row_end < p.T ? row_end : p.T;
  // first position of this wave's entries of expert e: the expert's offset, its entries in earlier workgroups and in
  // the earlier waves of this one (all loads independent of each other)
  for (int e = lane; e < E; e += 64) {
    int b = p.col_offs[e] + p.wg_prefix[(int64_t)blockIdx.x * E + e];
    int prev[kWaves - 1];
#pragma unroll
    for (int w = 0; w < kWaves - 1; ++w) prev[w] = w < wave ? p.partials[(int64_t)(blockIdx.x * kWaves + w) * E + e] : 0;
#pragma unroll
    for (int w = 0; w < kWaves - 1; ++w) b += prev[w];
    base_s[wave][e] = b;
  }
  wave_sync();
  const int64_t f_begin = (int64_t)row_begin * k, f_end = (int64_t)row_end * k;
  const int64_t n_valid = (int64_t)(n_rows < p.T ? n_rows : p.T) * k;
  const unsigned long long lt_mask = (1ull << lane) - 1ull;
  for (int64_t f0 = f_begin; f0 < f_end; f0 += 64) {
    const int64_t f = f0 + lane;
    const bool in = f < f_end;
    int e = -1;
    uint32_t gate_bits = 0;  // fetched together with the index: its latency is hidden behind the ranking below
    if (in && f < n_valid) {
      e = p.indx16 ? (int)p.indx16[f] : p.indx32[f];
      if (p.gammas_out) gate_bits = p.vals_bytes == 4 ? static_cast<const uint32_t*>(p.vals)[f] : (uint32_t) static_cast<const uint16_t*>(p.vals)[f];
    }
    const bool valid = e >= 0 && e < E;
    int pos = -1;
    unsigned long long todo = __ballot(valid);
    while (todo) {
      const int leader = __ffsll((long long)todo) - 1;
      const int e0 = __shfl(e, leader);
      const unsigned long long same = __ballot(valid && e == e0);
      if (valid && e == e0) pos = base_s[wave][e0] + __popcll(same & lt_mask);
      wave_sync();
      if (lane == leader) base_s[wave][e0] = base_s[wave][e0] + __popcll(same);
      wave_sync();
      todo &= ~same;
    }
    if (valid) {
      p.row_sorted[f] = pos;
      p.col_sorted[pos] = (int32_t)f;
      if (p.gather_out) p.gather_out[pos] = (int32_t)(f / k);
      if (p.gammas_out) {
        if (p.vals_bytes == 4)
          static_cast<uint32_t*>(p.gammas_out)[pos] = gate_bits;
        else
          static_cast<uint16_t*>(p.gammas_out)[pos] = (uint16_t)gate_bits;
      }
    }
  }
}

// Rows one wave routes: one for small batches (latency), more as T grows so that the workspace stays small: at most
// 1024 waves (512 when a row is long: E > 256), i.e. 256 / 128 rows of workgroup totals for the scan to walk.  A wave
// pays about 1.2 us per row (a dependent chain of lane exchanges, alone on its SIMD); with 2048 waves the scan's longer
// walk (512 rows: 16 us against 12) costs more than the shorter waves save.
int rows_per_wave_for(int T, int E) {
  const int64_t max_units = E <= 256 ? 1024 : 512;
  int rpw = 1;
  while ((int64_t)rpw * max_units < T) rpw *= 2;
  return rpw;
}

template <int DT>
int32_t launch_topk(const TopkParams& p, int units, hipStream_t st) {
  const int grid = (units + kWaves - 1) / kWaves;
  const int epl = (p.E + 63) / 64;
#define TK_EPL(N)                                                                                              \
  if (epl <= N) {                                                                                              \
    if (p.use_provided_indx)                                                                                   \
      hipLaunchKernelGGL((route_topk_kernel<DT, N, true>), dim3(grid), dim3(kWaves * 64), 0, st, p);           \
    else                                                                                                       \
      hipLaunchKernelGGL((route_topk_kernel<DT, N, false>), dim3(grid), dim3(kWaves * 64), 0, st, p);          \
    return check_launch("route_topk_kernel");                                                                  \
  }
  TK_EPL(1)
  TK_EPL(2)
  TK_EPL(4)
  TK_EPL(8)
  TK_EPL(16)
  TK_EPL(32)
#undef TK_EPL
  return fail(TK_ERR_UNSUPPORTED, "tk_route: more than %d experts", kMaxExperts);
}

template <int DT>
int32_t launch_small_dt(const SmallParams& q, hipStream_t st) {
  const int epl = (q.t.E + 63) / 64;
#define TK_EPL(N)                                                                                              \
  if (epl <= N) {                                                                                              \
    if (q.t.use_provided_indx)                                                                                 \
      hipLaunchKernelGGL((route_small_kernel<DT, N, true>), dim3(1), dim3(kScanThreads), 0, st, q);            \
    else                                                                                                       \
      hipLaunchKernelGGL((route_small_kernel<DT, N, false>), dim3(1), dim3(kScanThreads), 0, st, q);           \
    return check_launch("route_small_kernel");                                                                 \
  }
  TK_EPL(1)
  TK_EPL(2)
  TK_EPL(4)
  TK_EPL(8)
  TK_EPL(16)
  TK_EPL(32)
#undef TK_EPL
  return fail(TK_ERR_UNSUPPORTED, "tk_route: more than %d experts", kMaxExperts);
}

int32_t launch_small(const SmallParams& q, int dt, hipStream_t st) {
  if (dt == TK_BF16) return launch_small_dt<TK_BF16>(q, st);
  if (dt == TK_F16) return launch_small_dt<TK_F16>(q, st);
  return launch_small_dt<TK_F32>(q, st);
}

}  // namespace
}  // namespace tk

using namespace tk;

extern "C" int64_t tk_route_workspace_bytes(int32_t T, int32_t E) {
  if (T <= 0 || E <= 0) return 0;
  const int rpw = rows_per_wave_for(T, E);
  const int64_t units = (T + rpw - 1) / rpw;
  const int64_t units_pad = (units + kWaves - 1) / kWaves * kWaves;
  return (units_pad * E + units_pad / kWaves * E + (int64_t)E + 1) * 4;  // wave histograms, workgroup totals, expert offsets
}

// One routing pass with the kernels' scratch memory at `workspace` (tk_route_workspace_bytes(T, E) bytes, every word
// of which is written before it is read, so the memory may hold anything).
static int32_t route_impl(const tk_route_desc* d, void* workspace, tk_stream_t stream) {
  const int T = d->n_tokens, E = d->n_experts, k = d->k;
  if (T < 0 || E <= 0 || k <= 0) return fail(TK_ERR_INVALID, "tk_route: bad sizes T=%d E=%d k=%d", T, E, k);
  if (k > 64 || k > E) return fail(TK_ERR_INVALID, "tk_route: k=%d must be <= min(64, E)", k);
  if (E > kMaxExperts) return fail(TK_ERR_UNSUPPORTED, "tk_route: at most %d experts are supported (got %d)", kMaxExperts, E);
  if (T == 0) return TK_OK;
  const bool want_meta = d->col_sum != nullptr;
  if (!d->indx) return fail(TK_ERR_INVALID, "tk_route: indx buffer is required");
  if (!d->logits && !d->use_provided_indx) return fail(TK_ERR_INVALID, "tk_route: logits are required unless indices are provided");
  if (want_meta && (!d->col_sorted_indx || !d->row_sorted_indx || !workspace)) return fail(TK_ERR_INVALID, "tk_route: metadata outputs / workspace missing");
  if (d->indx_dtype != TK_I16) return fail(TK_ERR_UNSUPPORTED, "tk_route: indx must be int16");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int rpw = rows_per_wave_for(T, E);
  const int units = (T + rpw - 1) / rpw;
  const int units_pad = (units + kWaves - 1) / kWaves * kWaves;
  int32_t* partials = static_cast<int32_t*>(workspace);
  int32_t* wg_totals = partials ? partials + (int64_t)units_pad * E : nullptr;
  int32_t* col_offs = partials ? wg_totals + (int64_t)(units_pad / kWaves) * E : nullptr;

  TopkParams tp;
  tp.logits = d->logits;
  tp.stride_m = d->logits_stride_m;
  tp.T = T;
  tp.n_rows_imm = d->n_rows_ptr ? T : (d->n_rows < 0 ? T : d->n_rows);
  tp.n_rows_ptr = d->n_rows_ptr;
  tp.E = E;
  tp.k = k;
  tp.apply_softmax = d->apply_softmax;
  tp.use_provided_indx = d->use_provided_indx;
  tp.vals = d->vals;
  tp.indx = static_cast<int16_t*>(d->indx);
  tp.bitmatrix = static_cast<uint32_t*>(d->bitmatrix);
  tp.bm_stride_w = d->bitmatrix_stride_w;
  tp.partials = want_meta ? partials : nullptr;
  tp.wg_totals = want_meta ? wg_totals : nullptr;
  tp.rows_per_wave = rpw;
  tp.fill_a = want_meta ? d->col_sorted_indx : nullptr;
  tp.fill_b = want_meta ? d->row_sorted_indx : nullptr;
  tp.fill_c = want_meta ? d->gather_indx : nullptr;
  if ((int64_t)T * k <= kSmallCut) {
    // small batch: the whole pass in one launch
    SmallParams sq;
    sq.t = tp;
    sq.t.partials = nullptr;
    sq.t.fill_a = sq.t.fill_b = sq.t.fill_c = nullptr;
    sq.col_sum = want_meta ? d->col_sum : nullptr;
    sq.col_offs = col_offs;
    sq.col_sorted = d->col_sorted_indx;
    sq.row_sorted = d->row_sorted_indx;
    sq.gather_out = d->gather_indx;
    sq.gammas_out = d->vals ? d->gammas : nullptr;
    sq.vals_bytes = (d->logits_dtype == TK_F32 || !d->logits) ? 4 : 2;
    sq.want_ragged = d->slice_offs != nullptr;
    sq.r.slice_offs = d->slice_offs;
    sq.r.block_offs = d->block_offs;
    sq.r.block_offs_stride = d->block_offs_stride;
    sq.r.block_sched = d->block_schedule;
    sq.r.block_sched_stride = d->block_schedule_stride;
    sq.r.max_n_blocks = d->max_n_blocks;
    if (want_meta && sq.want_ragged && (!d->block_offs || (!d->block_schedule && d->max_n_blocks > 0))) return fail(TK_ERR_INVALID, "tk_route: incomplete ragged outputs");
    if (d->logits && d->logits_dtype != TK_F32 && d->logits_dtype != TK_BF16 && d->logits_dtype != TK_F16) return fail(TK_ERR_UNSUPPORTED, "tk_route: logits dtype %d", d->logits_dtype);
    return launch_small(sq, d->logits ? d->logits_dtype : TK_F32, st);
  }
  int32_t rc;
  if (d->logits_dtype == TK_F32 || !d->logits)
    rc = launch_topk<TK_F32>(tp, units, st);
  else if (d->logits_dtype == TK_BF16)
    rc = launch_topk<TK_BF16>(tp, units, st);
  else if (d->logits_dtype == TK_F16)
    rc = launch_topk<TK_F16>(tp, units, st);
  else
    return fail(TK_ERR_UNSUPPORTED, "tk_route: logits dtype %d", d->logits_dtype);
  if (rc != TK_OK || !want_meta) return rc;

  RaggedOut ro;
  ro.slice_offs = d->slice_offs;
  ro.block_offs = d->block_offs;
  ro.block_offs_stride = d->block_offs_stride;
  ro.block_sched = d->block_schedule;
  ro.block_sched_stride = d->block_schedule_stride;
  ro.max_n_blocks = d->max_n_blocks;
  const int want_ragged = d->slice_offs != nullptr;
  if (want_ragged && (!d->block_offs || (!d->block_schedule && d->max_n_blocks > 0))) return fail(TK_ERR_INVALID, "tk_route: incomplete ragged outputs");
  hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(kScanThreads), 0, st, wg_totals, units_pad / kWaves, E, d->col_sum, col_offs, want_ragged, ro);
  rc = check_launch("route_scan_kernel");
  if (rc != TK_OK) return rc;

  ScatterParams sp;
  sp.indx16 = static_cast<const int16_t*>(d->indx);
  sp.indx32 = nullptr;
  sp.T = T;
  sp.k = k;
  sp.E = E;
  sp.n_rows_imm = tp.n_rows_imm;
  sp.n_rows_ptr = d->n_rows_ptr;
  sp.rows_per_wave = rpw;
  sp.partials = partials;
  sp.wg_prefix = wg_totals;
  sp.col_offs = col_offs;
  sp.col_sorted = d->col_sorted_indx;
  sp.row_sorted = d->row_sorted_indx;
  sp.gather_out = d->gather_indx;
  sp.vals = d->vals;
  sp.gammas_out = d->vals ? d->gammas : nullptr;
  sp.vals_bytes = (d->logits_dtype == TK_F32 || !d->logits) ? 4 : 2;
  hipLaunchKernelGGL(route_scatter_kernel, dim3(units_pad / kWaves), dim3(kWaves * 64), 0, st, sp);
  return check_launch("route_scatter_kernel");
}

extern "C" int32_t tk_route(const tk_route_desc* d, tk_stream_t stream) {
  if (!d) return fail(TK_ERR_INVALID, "tk_route: null descriptor");
  return route_impl(d, d->workspace, stream);
}

// ---- routing without any allocation: the workspace is a device array owned by the library ------------------
// `route_scratch` exists once per GPU the library runs on and lives until the process ends.  Host code never
// passes the array's name to a kernel (on the host it is a stand-in, not a device address): the address on the
// current device is looked up once per device with hipGetSymbolAddress and kept in `g_route_scratch`.
constexpr int64_t kRouteScratchBytes = TK_ROUTE_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char route_scratch[kRouteScratchBytes];

static std::mutex g_route_scratch_mu;
static void* g_route_scratch[64];  // per device id, filled under the mutex

static int32_t route_scratch_ptr(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(TK_ERR_LAUNCH, "tk_route_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= 64) return fail(TK_ERR_UNSUPPORTED, "tk_route_static: device id %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_route_scratch_mu);
  if (!g_route_scratch[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(route_scratch));
    if (e != hipSuccess || !ptr) return fail(TK_ERR_LAUNCH, "tk_route_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_route_scratch[dev] = ptr;
  }
  *out = g_route_scratch[dev];
  return TK_OK;
}

extern "C" int32_t tk_route_static_prepare(void) {
  void* ws = nullptr;
  return route_scratch_ptr(&ws);
}

extern "C" int32_t tk_route_static(const tk_route_desc* d, tk_stream_t stream) {
  if (!d) return fail(TK_ERR_INVALID, "tk_route_static: null descriptor");
  const int64_t need = tk_route_workspace_bytes(d->n_tokens, d->n_experts);
  if (need > kRouteScratchBytes)
    return fail(TK_ERR_UNSUPPORTED, "tk_route_static: %d tokens x %d experts need %lld bytes of scratch, the built-in buffer holds %lld; use tk_route with a caller workspace",
                d->n_tokens, d->n_experts, (long long)need, (long long)kRouteScratchBytes);
  void* ws = nullptr;
  if (const int32_t rc = route_scratch_ptr(&ws)) return rc;
  return route_impl(d, ws, stream);
}

extern "C" int32_t tk_ragged_metadata(const int32_t* slice_sizes, int32_t n_slices, int32_t* slice_offs, int32_t* block_offs,
                                      int64_t block_offs_stride, int32_t* block_schedule, int64_t block_schedule_stride,
                                      int32_t max_n_blocks, tk_stream_t stream) {
  if (n_slices < 0 || max_n_blocks < 0) return fail(TK_ERR_INVALID, "tk_ragged_metadata: negative size");
  if (n_slices >= 65536) return fail(TK_ERR_INVALID, "tk_ragged_metadata: at most 65535 slices");
  if (!slice_offs || !block_offs || (!block_schedule && max_n_blocks > 0) || (!slice_sizes && n_slices > 0)) return fail(TK_ERR_INVALID, "tk_ragged_metadata: null pointer");
  RaggedOut ro;
  ro.slice_offs = slice_offs;
  ro.block_offs = block_offs;
  ro.block_offs_stride = block_offs_stride;
  ro.block_sched = block_schedule;
  ro.block_sched_stride = block_schedule_stride;
  ro.max_n_blocks = max_n_blocks;
  hipLaunchKernelGGL(ragged_metadata_kernel, dim3(1), dim3(kScanThreads), 0, static_cast<hipStream_t>(stream), slice_sizes, n_slices, ro);
  return check_launch("ragged_metadata_kernel");
}

extern "C" int32_t tk_ragged_remap(const int32_t* slice_sizes, const int32_t* slice_offs, const int32_t* block_offs,
                                   int64_t block_offs_stride, const int32_t* block_schedule, int64_t block_schedule_stride,
                                   const int32_t* slice_map, int32_t n_slices, int32_t n_block_sizes, int32_t max_n_blocks,
                                   int32_t* slice_sizes_out, int32_t* slice_offs_out, int32_t* block_offs_out,
                                   int64_t block_offs_out_stride, int32_t* block_schedule_out, int64_t block_schedule_out_stride,
                                   tk_stream_t stream) {
  if (n_slices < 0 || n_block_sizes < 0 || max_n_blocks < 0) return fail(TK_ERR_INVALID, "tk_ragged_remap: negative size");
  if (n_slices >= 65536) return fail(TK_ERR_INVALID, "tk_ragged_remap: at most 65535 slices");
  if (!slice_offs || !slice_offs_out || (n_slices > 0 && (!slice_sizes || !slice_map || !slice_sizes_out)) ||
      (n_block_sizes > 0 && (!block_offs || !block_offs_out)) || (n_block_sizes > 0 && max_n_blocks > 0 && (!block_schedule || !block_schedule_out)))
    return fail(TK_ERR_INVALID, "tk_ragged_remap: null pointer");
  RemapParams p;
  p.slice_sizes = slice_sizes;
  p.slice_offs = slice_offs;
  p.block_offs = block_offs;
  p.block_offs_stride = block_offs_stride;
  p.block_sched = block_schedule;
  p.block_sched_stride = block_schedule_stride;
  p.slice_map = slice_map;
  p.n_slices = n_slices;
  p.max_n_blocks = max_n_blocks;
  p.slice_sizes_out = slice_sizes_out;
  p.slice_offs_out = slice_offs_out;
  p.block_offs_out = block_offs_out;
  p.block_offs_out_stride = block_offs_out_stride;
  p.block_sched_out = block_schedule_out;
  p.block_sched_out_stride = block_schedule_out_stride;
  hipLaunchKernelGGL(ragged_remap_kernel, dim3(1 + n_block_sizes), dim3(kScanThreads), 0, static_cast<hipStream_t>(stream), p);
  return check_launch("ragged_remap_kernel");
}

extern "C" int32_t tk_topk_backward(const void* x, int32_t dtype, int64_t stride_xm, const int16_t* indx, int64_t stride_im, const void* dy,
                                    int64_t stride_dym, void* dx, int64_t stride_dxm, int32_t n_tokens, int32_t n_experts, int32_t k,
                                    int32_t apply_softmax, int32_t n_rows, const int32_t* n_rows_ptr, tk_stream_t stream) {
  if (n_tokens < 0 || n_experts <= 0 || k <= 0 || k > 64) return fail(TK_ERR_INVALID, "tk_topk_backward: bad sizes T=%d E=%d k=%d", n_tokens, n_experts, k);
  if (n_tokens == 0) return TK_OK;
  if (!x || !indx || !dy || !dx) return fail(TK_ERR_INVALID, "tk_topk_backward: null pointer");
  const int rows = n_rows < 0 ? n_tokens : n_rows;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)((n_tokens + 3) / 4));
#define TK_TB(D)                                                                                                                   \
  if (dtype == D) {                                                                                                                \
    hipLaunchKernelGGL(topk_backward_kernel<D>, grid, dim3(256), 0, st, x, stride_xm, indx, stride_im, dy, stride_dym, dx, stride_dxm, \
                       n_tokens, n_experts, k, apply_softmax, rows, n_rows_ptr);                                                   \
    return check_launch("topk_backward_kernel");                                                                                  \
  }
  TK_TB(TK_F32)
  TK_TB(TK_BF16)
  TK_TB(TK_F16)
#undef TK_TB
  return fail(TK_ERR_UNSUPPORTED, "tk_topk_backward: dtype %d", dtype);
}
