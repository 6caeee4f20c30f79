#include "gemm_common.h"

namespace tk {
namespace {

// ------------------------------------------------------------------------------------------------
// MXFP4 weights in the tile-native layout, decode shapes (block_m 16 / 32): a pure weight stream
// ------------------------------------------------------------------------------------------------
// A few rows per expert: the kernel is bound by reading each active expert's weights once.  Every wave works
// alone (no LDS, no barrier): it owns one 32-column weight fragment of one row block, streams the fragment's
// K-stages through a four-deep register ring (8 KiB in flight per wave, twelve to sixteen waves per CU), reads its
// rows' activations straight from L2 through a ring of the same depth (each lane 64 contiguous bytes per stage;
// one stage ahead left their latency exposed), and issues 16x16x32 MFMAs
// transposed like the prefill kernel (lane = column, 4 k-groups).  Within a stage lane group kg owns
// k in [kg*32, kg*32 + 32): exactly one MX block and one 16-byte piece of the tiled layout.
// Epilogue of the decode kernel with the top-k combine fused behind the scatter (the reference runs `reduce` over the k
// rows of every token as a launch of its own, reduce.py:1143-1165).  The k rows of token t are written by up to k
// different waves, anywhere on the chip; each counts itself in at counter (t, fragment) once its rows have reached
// memory, and the wave that arrives last sums the k rows in their order j = 0..k-1 in fp32, exactly as the
// stand-alone kernel does, writes the token's row of the result and clears the counter for the next launch.
// The eight XCDs have an L2 each, so rows that another XCD will read go around it: stores and loads of y carry the
// sc0 sc1 cache policy (write-through to memory / read from memory) and the counter is a device-scope atomic; the
// alternative, a device-scope release fence per wave, writes back and invalidates a whole L2 each time and more than
// doubled the kernel's time.  acc[g][j][i]: sub-fragment g (columns F*32 + g*16 + kg*4 + i), row fragment j.
// Operands of the combine epilogue that do not depend on the accumulators; the kernel fetches them before its K loop
// so that their latency is not part of every wave's tail.
template <int MR, int NFD>
struct CombineOperands {
  float gam[MR];
  int dst[MR];          // destination row (flat position t * k + j) or -1
  float b4[NFD][2][4];  // bias of the lane's columns
};

template <int MR, int NFD>
__device__ __forceinline__ CombineOperands<MR, NFD> load_combine_operands(const GemmParams& p, int expert, int off_m, int start_m, int eM,
                                                                          const int (&F)[NFD], int lr, int kg) {
  CombineOperands<MR, NFD> o;
  const int N = p.N;
#pragma unroll
  for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = F[fd] * 32 + g * 16 + kg * 4 + i;
        o.b4[fd][g][i] = (p.bias && n < N) ? load_scalar(p.bias, (int64_t)expert * p.bias_stride_e + n, p.bias_is_f32) : 0.f;
      }
#pragma unroll
  for (int j = 0; j < MR; ++j) {
    const int row = off_m + j * 16 + lr;
    const bool ok = row < eM;
    const int srow = start_m + (ok ? row : eM - 1);
    o.gam[j] = p.gammas ? load_scalar(p.gammas, srow, p.gammas_is_f32) : 1.0f;
    const int dst = srow < p.scatter_len ? p.scatter[srow] : -1;
    o.dst[j] = ok ? dst : -1;
  }
  return o;
}

// The NFD fragments of a wave go through every step together (all stores, one wait, all counters, all loads), so the
// chain of memory round trips at the end of a wave is as long for two fragments as for one.
template <int MR, int NFD>
__device__ __forceinline__ void combine_epilogue(const GemmParams& p, f32x4_t (&acc)[NFD][2][MR], const CombineOperands<MR, NFD>& o,
                                                 const int (&F)[NFD], const bool (&live_f)[NFD], int nfr, int lr, int kg) {
  constexpr int kThrough = 1 | 16;  // aux bits of the buffer instructions: sc0 | sc1
  const int N = p.N, k = p.combine_k;
  const __amdgpu_buffer_rsrc_t yrsrc = __builtin_amdgcn_make_buffer_rsrc(p.y, 0, p.y_bytes, 0x00020000);
  const uint32_t row_bytes = (uint32_t)(p.y_stride_m * 2);
  int token[MR];
#pragma unroll
  for (int j = 0; j < MR; ++j) {
    const int dst = o.dst[j];
    const float gam = o.gam[j];
    token[j] = dst >= 0 ? dst / k : -1;
#pragma unroll
    for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        const int n0 = F[fd] * 32 + g * 16 + kg * 4;
        const u32x2_t w = {pack_bf16x2((acc[fd][g][j][0] + o.b4[fd][g][0]) * gam, (acc[fd][g][j][1] + o.b4[fd][g][1]) * gam),
                           pack_bf16x2((acc[fd][g][j][2] + o.b4[fd][g][2]) * gam, (acc[fd][g][j][3] + o.b4[fd][g][3]) * gam)};
        const uint32_t off = (live_f[fd] && dst >= 0 && n0 < N) ? (uint32_t)dst * row_bytes + (uint32_t)n0 * 2u : kDroppedStore;
        __builtin_amdgcn_raw_buffer_store_b64(w, yrsrc, off, 0, kThrough);
      }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's rows have reached memory before it is counted
  bool last[MR][NFD];
#pragma unroll
  for (int j = 0; j < MR; ++j)
#pragma unroll
    for (int fd = 0; fd < NFD; ++fd) {
      int seen = -1;
      if (kg == 0 && token[j] >= 0 && live_f[fd])
        seen = __hip_atomic_fetch_add(&p.combine_counters[(int64_t)token[j] * nfr + F[fd]], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      seen = __shfl(seen, lr);  // the row's four lanes (lr, lr + 16, ...) share lane lr's count
      last[j][fd] = token[j] >= 0 && live_f[fd] && seen == k - 1;
    }
  // (the loads below depend on the atomics' results, so they cannot be issued before those have been performed)
#pragma unroll
  for (int j = 0; j < MR; ++j)
#pragma unroll
    for (int fd = 0; fd < NFD; ++fd) {
      const uint32_t base = last[j][fd] ? (uint32_t)(token[j] * k) * row_bytes : kDroppedStore;
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        const int n0 = F[fd] * 32 + g * 16 + kg * 4;
        float sum[4] = {0.f, 0.f, 0.f, 0.f};
        for (int jj = 0; jj < k; ++jj) {
          const uint32_t off = (last[j][fd] && n0 < N) ? base + (uint32_t)jj * row_bytes + (uint32_t)n0 * 2u : kDroppedStore;
          const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(yrsrc, off, 0, kThrough);  // out-of-range lanes read zero
          sum[0] += bits_f32(v.x << 16);
          sum[1] += bits_f32(v.x & 0xFFFF0000u);
          sum[2] += bits_f32(v.y << 16);
          sum[3] += bits_f32(v.y & 0xFFFF0000u);
        }
        if (last[j][fd] && n0 < N) {
          uint16_t* out = p.combine_out + (int64_t)token[j] * p.combine_stride + n0;
          if (n0 + 4 <= N && (p.combine_stride & 3) == 0) {
            *reinterpret_cast<uint2*>(out) = make_uint2(pack_bf16x2(sum[0], sum[1]), pack_bf16x2(sum[2], sum[3]));
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (n0 + i < N) out[i] = f32_to_bf16_bits(sum[i]);
          }
        }
      }
      if (last[j][fd] && kg == 0)
        __hip_atomic_store(&p.combine_counters[(int64_t)token[j] * nfr + F[fd]], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ONCE: the whole problem is one row block per slice (at most 16 rows in all), so every weight byte is read exactly
// once and is fetched with the non-temporal hint; several row blocks of a slice share its fragments through the L2.
template <int MR, int NFD, bool SWIGLU, bool ONCE = false>
__global__ __launch_bounds__(256) void moe_gemm_mxd_kernel(const GemmParams p) {
  typedef Frag<16> FR;
  constexpr int WDD = 4, XDD = 4;  // ring depths (stages) of the weight / activation registers (both run 3 stages ahead)
  __shared__ float red[3][NFD * 2 * MR * 4][64];  // K-split partial sums of waves 1..3
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, kg = lane >> 4;
  const int K = p.K, N = p.N;
  const int nst = p.w_nst;
  const int nfr = (N + 31) >> 5;
  // A wave owns NFD neighbouring 32-column fragments of one row block: the activations it fetches (twice the bytes of a
  // fragment's weights per stage) then feed NFD fragments' MFMAs.
  const int nslot = (nfr + NFD - 1) / NFD;  // fragment groups per row block

  // K-split: when few tiles are live (a handful of active experts), 2 or 4 waves share a fragment group and take
  // every 2nd / 4th K-stage each, so that enough loads are in flight to cover the HBM latency.  The factor is
  // derived on the device from the live block count (the host never reads it) and is uniform over the grid;
  // the grid is launched for the largest factor and the surplus workgroups leave at once.
  const int nblk = p.slice_sizes ? p.block_offs[p.n_slices] : p.total_tiles;
  const int frag_tiles = nblk * nslot;  // (row block, fragment group) pairs = waves at split 1
  const int ksplit = frag_tiles <= 1024 ? 4 : (frag_tiles <= 2048 ? 2 : 1);
  const int fpw = 4 / ksplit;                        // fragment groups per workgroup
  const int grid_n = (nslot + fpw - 1) / fpw;        // workgroups per row block
  // Workgroups go round-robin to the 8 XCDs.  With the row blocks a multiple of 8 workgroups apart, the workgroups that
  // read one weight fragment for the different row blocks of an expert (an expert with more rows than a block holds)
  // land on ONE XCD, close together in time, and share the fragment through its L2 instead of fetching it again.
  const int grid_n8 = (grid_n + 7) & ~7;
  if ((int)blockIdx.x >= nblk * grid_n8) return;
  const int pid_n = blockIdx.x % grid_n8, pid_m = blockIdx.x / grid_n8;
  if (pid_n >= grid_n) return;
  const int kslice = wave % ksplit;
  int expert, off_m, start_m, eM;
  if (p.slice_sizes) {
    const int sched = p.block_sched[pid_m];
    expert = sched & 0xFFFF;
    off_m = (sched >> 16) * (MR * 16);
    start_m = p.slice_offs[expert];
    eM = p.slice_sizes[expert];
  } else {
    expert = 0;
    off_m = pid_m * (MR * 16);
    start_m = 0;
    eM = p.M;
  }
  const int slot = pid_n * fpw + wave / ksplit;  // this wave's fragment group
  const bool live_wave = slot < nslot;
  int F[NFD];
  bool live_f[NFD];
#pragma unroll
  for (int fd = 0; fd < NFD; ++fd) {
    const int f = (live_wave ? slot : nslot - 1) * NFD + fd;
    live_f[fd] = live_wave && f < nfr;
    F[fd] = f < nfr ? f : nfr - 1;
  }
  const int rows = (eM - off_m) < MR * 16 ? (eM - off_m) : MR * 16;
  const int nj = (rows + 15) >> 4;  // row fragments with valid rows (1..MR)
  // this wave's stages: kslice, kslice + ksplit, ...
  const int my_nst = (nst - kslice + ksplit - 1) / ksplit;

  // weights: sub-fragment g holds columns F*32 + g*16 + lr; this lane's piece of a stage is k-block kg
  const uint8_t* wbase[NFD];
  const uint8_t* sbase[NFD];
#pragma unroll
  for (int fd = 0; fd < NFD; ++fd) {
    wbase[fd] = p.w + (int64_t)expert * p.w_stride_e + (int64_t)F[fd] * nst * 2048 + (kg & 1) * 1024 + ((kg >> 1) * 32 + lr) * 16;
    sbase[fd] = p.w_scale + (int64_t)expert * p.ws_stride_e + (int64_t)F[fd] * nst * 128 + lr * 4;
  }
  // activations: row j*16 + lr, 64 bytes per stage at k offset kg*32
  const uint8_t* xptr[MR];
#pragma unroll
  for (int j = 0; j < MR; ++j) {
    int row = off_m + j * 16 + lr;
    row = row < eM ? row : eM - 1;
    const int64_t src = p.gather ? (int64_t)p.gather[start_m + row] : (int64_t)(start_m + row);
    xptr[j] = p.x + src * p.x_stride_m * 2;
  }

  typename FR::acc_t acc[NFD][2][MR];
#pragma unroll
  for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int j = 0; j < MR; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[fd][g][j][i] = 0.f;

  u32x4_t wr[WDD][NFD][2];
  uint32_t sr[WDD][NFD][2];
  u32x4_t xr[XDD][MR][4];

  // `i` counts this wave's own stages; the global stage is kslice + i*ksplit (clamped: surplus loads re-read
  // the last stage and are never used)
  auto load_w = [&](auto slot_c, int i) __attribute__((always_inline)) {
    constexpr int SL = decltype(slot_c)::value;
    int s = kslice + i * ksplit;
    s = s < nst ? s : nst - 1;
#pragma unroll
    for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        const u32x4_t* wp = reinterpret_cast<const u32x4_t*>(wbase[fd] + (int64_t)s * 2048 + g * 256);
        const uint32_t* sp = reinterpret_cast<const uint32_t*>(sbase[fd] + (int64_t)s * 128 + g * 64);
        if constexpr (ONCE) {
          wr[SL][fd][g] = __builtin_nontemporal_load(wp);
          sr[SL][fd][g] = __builtin_nontemporal_load(sp);
        } else {
          wr[SL][fd][g] = *wp;
          sr[SL][fd][g] = *sp;
        }
      }
  };
  auto load_x = [&](auto slot_c, int i) __attribute__((always_inline)) {
    constexpr int SL = decltype(slot_c)::value;
    const int s = kslice + i * ksplit;
#pragma unroll
    for (int j = 0; j < MR; ++j)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        int k0 = s * 128 + kg * 32 + t * 8;
        k0 = k0 < K - 8 ? k0 : K - 8;  // past K the padded weights are zero; any finite activation will do
        xr[SL][j][t] = *reinterpret_cast<const u32x4_t*>(xptr[j] + k0 * 2);
      }
  };
  auto compute = [&](auto wslot_c, auto xslot_c) __attribute__((always_inline)) {
    constexpr int WS = decltype(wslot_c)::value;
    constexpr int XS = decltype(xslot_c)::value;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      bf16x8_t wf[NFD][2];
#pragma unroll
      for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          const u32x4_t v = wr[WS][fd][g];
          const uint32_t raw = t == 0 ? v.x : t == 1 ? v.y : t == 2 ? v.z : v.w;
          wf[fd][g] = dequant8(raw, bits_f32(((sr[WS][fd][g] >> (8 * kg)) & 0xFFu) << 23));
        }
#pragma unroll
      for (int j = 0; j < MR; ++j) {
        if (j < nj) {
          const bf16x8_t xf = __builtin_bit_cast(bf16x8_t, xr[XS][j][t]);
#pragma unroll
          for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
            for (int g = 0; g < 2; ++g) acc[fd][g][j] = FR::mma(wf[fd][g], xf, acc[fd][g][j]);
        }
      }
    }
  };

  CombineOperands<MR, NFD> cops;
  bool combine = false;
  if constexpr (!SWIGLU) {
    combine = p.combine_k > 0;
    if (combine && live_wave && kslice == 0) cops = load_combine_operands<MR, NFD>(p, expert, off_m, start_m, eM, F, lr, kg);
  }
  if (live_wave) {
    // prologue: fill the rings in the order the steady state leaves them (weights run WDD-1 stages ahead,
    // activations XDD-1)
    static_for<0, WDD - 1>([&](auto c_c) __attribute__((always_inline)) {
      constexpr int c = decltype(c_c)::value;
      load_w(c_c, c);
      if constexpr (c < XDD - 1) load_x(c_c, c);
    });
    int c = 0;
    for (; c + WDD - 1 < my_nst; c += WDD) {
      static_for<0, WDD>([&](auto i_c) __attribute__((always_inline)) {
        constexpr int i = decltype(i_c)::value;
        load_w(template_int<(i + WDD - 1) % WDD>{}, c + i + WDD - 1);
        load_x(template_int<(i + XDD - 1) % XDD>{}, c + i + XDD - 1);
        compute(i_c, template_int<i % XDD>{});
      });
    }
    static_for<0, WDD - 1>([&](auto i_c) __attribute__((always_inline)) {
      constexpr int i = decltype(i_c)::value;
      if (c + i < my_nst) {
        load_x(template_int<(i + XDD - 1) % XDD>{}, c + i + XDD - 1);
        compute(i_c, template_int<i % XDD>{});
      }
    });
  }
  if (ksplit > 1) {
    // sum the K-slices of a fragment group in the wave with kslice 0 (through LDS), which then runs the epilogue
    if (kslice != 0) {
#pragma unroll
      for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
        for (int g = 0; g < 2; ++g)
#pragma unroll
          for (int j = 0; j < MR; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave - 1][((fd * 2 + g) * MR + j) * 4 + i][lane] = acc[fd][g][j][i];
    }
    __syncthreads();
    if (kslice != 0) return;
    for (int o = 1; o < ksplit; ++o)
#pragma unroll
      for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
        for (int g = 0; g < 2; ++g)
#pragma unroll
          for (int j = 0; j < MR; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[fd][g][j][i] += red[wave + o - 1][((fd * 2 + g) * MR + j) * 4 + i][lane];
  }
  if constexpr (!SWIGLU) {
    if (combine) {
      if (live_wave) combine_epilogue<MR, NFD>(p, acc, cops, F, live_f, nfr, lr, kg);
      return;
    }
  }
#pragma unroll
  for (int fd = 0; fd < NFD; ++fd) {
    if (!live_f[fd]) continue;
    gemm_epilogue<16, 1, MR, 2, SWIGLU>(p, acc[fd], expert, off_m, start_m, eM, F[fd] * 32, F[fd] * 32 + 32 <= N, 0, lr, kg);
  }
}

template <int MR, int NFD, bool ONCE = false>
int32_t launch_mxd_n(const GemmParams& p, int grid_m, bool swiglu, hipStream_t st) {
  GemmParams q = p;
  q.total_tiles = grid_m;  // row blocks in the non-ragged case
  // sized for a K-split of 4 (one fragment group per workgroup); with a smaller split the surplus leaves at once
  const int64_t grid = (int64_t)grid_m * ((cdiv(cdiv(p.N, 32), NFD) + 7) & ~int64_t(7));
  if (grid <= 0) return TK_OK;
  if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: grid too large");
  if (swiglu)
    hipLaunchKernelGGL((moe_gemm_mxd_kernel<MR, NFD, true, ONCE>), dim3((unsigned)grid), dim3(256), 0, st, q);
  else
    hipLaunchKernelGGL((moe_gemm_mxd_kernel<MR, NFD, false, ONCE>), dim3((unsigned)grid), dim3(256), 0, st, q);
  return check_launch("moe_gemm_mxd_kernel");
}
template <int MR>
int32_t launch_mxd(const GemmParams& p, int grid_m, bool swiglu, hipStream_t st) {
  // Two fragments per wave halve the activation reads (which come from L2) at the price of half as many waves.  With
  // few rows only a few experts are live and the kernel needs every wave it can get to keep HBM busy; from about a
  // hundred rows on the activation traffic is what limits it.  (Measured at 128 experts, top-4: 16 tokens are 6 %
  // faster with one fragment, 64 tokens 8 % faster with two.)
  if constexpr (MR == 1)
    if (p.M <= 16) return launch_mxd_n<1, 1, true>(p, grid_m, swiglu, st);
  return p.M >= 128 ? launch_mxd_n<MR, 2>(p, grid_m, swiglu, st) : launch_mxd_n<MR, 1>(p, grid_m, swiglu, st);
}

}  // namespace

int32_t gemm_launch_mxd(const GemmParams& p, int block_m, int grid_m, bool swiglu, hipStream_t st) {
  if (block_m == 16) return launch_mxd<1>(p, grid_m, swiglu, st);
  return launch_mxd<2>(p, grid_m, swiglu, st);
}

}  // namespace tk
