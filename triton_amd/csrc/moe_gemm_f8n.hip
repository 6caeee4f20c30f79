#include "gemm_common.h"

namespace tk {
namespace {

// ------------------------------------------------------------------------------------------------
// e4m3 weights in a tile-native layout x e4m3 activations (prefill): FP8 MFMA, no conversion in the loop
// ------------------------------------------------------------------------------------------------
// Weight layout (built once per model by the host from the K-contiguous form): per expert, per fragment F of 32
// output columns (N padded to 32), per K-block s of 128 (K padded to 256 with zero weights, so the number of
// blocks is even): one 4 KiB block [q:4][lane:64][16 B]; lane = h*32 + lr holds the e4m3 bytes of column
// F*32 + lr for k in [s*128 + (q/2)*64 + h*32 + (q%2)*16, +16): pieces 2t and 2t+1 of a lane are the 32 consecutive
// bytes it feeds to the v_mfma_f32_32x32x64_f8f6f4 of K-step t.  The activation rows (gathered, one byte per
// element) are staged through LDS and read back as the same 32 consecutive bytes per lane, so both operands put
// the same k in the same byte position whatever order the instruction sums them in.  Per-row and per-column
// fp32 scales, bias, activation and gate weight are applied by the shared epilogue.
//
// Structure as in the MXFP4 prefill kernel: four waves, each owning NFW column fragments whose weights go
// global memory -> register double buffer -> MFMA, all sharing the MFW row fragments of the tile through an LDS
// double buffer; persistent grid with XCD-aware rounds and (expert, column tile, row block) tile order.  A stage
// is 256 bytes of K = four K-steps of 64, one workgroup barrier per stage (in step 3); the 64 memory instructions
// of a stage (LDS reads of the next step's activations, LDS writes of the next stage's activations with the
// refill of their staging registers, weight loads of the next stage) are dealt two or three to each of the 32
// MFMA slots: a slot that issues many loads back to back holds up the next MFMA.
template <int BLKM, int MFW, int NFW, bool SWIGLU>
__global__ __launch_bounds__(256) void moe_gemm_f8n_kernel(const GemmParams p) {
  typedef Frag<32> FR;
  constexpr int FM = 32, BM = MFW * 32, BN = 128 * NFW, KC = 256, NS = 4;
  constexpr int XPITCH = KC + 16;
  constexpr int XBYTES = BM * XPITCH;
  constexpr int XCH = 2 * MFW;  // 16-byte activation pieces per thread per stage
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int nw = __builtin_amdgcn_readfirstlane(tid >> 6);  // column quarter of the tile
  const int lr = lane & 31, h = lane >> 5;
  const int K = p.K, N = p.N;
  const int nst = p.w_nst;  // stages of 256 (two 4 KiB weight blocks per column fragment each)
  const int live = p.slice_sizes ? p.block_offs[p.n_slices] * p.grid_n : p.total_tiles;
  __shared__ int next_tile_s[2];  // written by thread 0 before a tile's first barrier: the id of the tile after it
  int tile_par = 0, n_tile = 0;
  // (claiming needs at least one workgroup per XCD queue: a queue's tiles are reached through the workgroups that
  // start on it.  With many rounds, or tiles that divide evenly among the workgroups, the static rounds are kept: a
  // partly filled last round then costs little, while tiles that start together walk K in step and find each other's
  // operands in the XCD's L2 — 4 % faster at 8192 tokens x top-2 of 8 experts, 56 rounds.)
  const bool dyn = p.tile_counters != nullptr && gridDim.x >= 8 && live % (int)gridDim.x != 0 && live < 32 * (int)gridDim.x;
  TileClaimer claimer;
  int pid = claimer.init(p.tile_counters, live), round0 = 0;
  // (dynamic: a workgroup whose queue is shorter than its first index gets no tile at all, which only happens when
  // there are fewer tiles than workgroups; its first two tiles are fixed, later ones are claimed)
  const int pid_second = claimer.second();
  if (!dyn) {
    const int in_round0 = live < (int)gridDim.x ? live : (int)gridDim.x;
    pid = (int)blockIdx.x < in_round0 ? xcd_remap(blockIdx.x, in_round0) : -1;
  }
  while (pid >= 0) {
  const bool claim_now = dyn && (n_tile >= 1 || pid_second < 0);
  if (claim_now) claimer.issue();  // the next tile's claim travels while this tile's first loads do
  int expert, blk_off, start_m, eM, pid_n;
  if (p.slice_sizes) {
    expert = p.block_sched[pid / p.grid_n] & 0xFFFF;
    const int first = p.block_offs[expert];
    const int nb = p.block_offs[expert + 1] - first;
    const int local = pid - first * p.grid_n;
    pid_n = local / nb;
    blk_off = (local - pid_n * nb) * BLKM;
    start_m = p.slice_offs[expert];
    eM = p.slice_sizes[expert];
  } else {
    pid_n = pid % p.grid_n;
    expert = 0;
    blk_off = (pid / p.grid_n) * BLKM;
    start_m = 0;
    eM = p.M;
  }
  const int blk_rows = (eM - blk_off) < BLKM ? (eM - blk_off) : BLKM;
  for (int pass_off = 0; pass_off < blk_rows; pass_off += BM) {
  const int off_m = blk_off + pass_off;
  const int rows = (blk_rows - pass_off) < BM ? (blk_rows - pass_off) : BM;
  const int nj = (rows + FM - 1) / FM;  // row fragments that hold valid rows (1..MFW)

  // ---- activation staging: piece j of this thread = row 16 j + tid/16, 16-byte chunk tid%16 of the stage ----
  const int xc = tid & 15;
  const uint8_t* xptr[XCH];
#pragma unroll
  for (int j = 0; j < XCH; ++j) {
    int row = off_m + (tid >> 4) + 16 * j;
    row = row < eM ? row : eM - 1;
    const int64_t src = p.gather ? (int64_t)p.gather[start_m + row] : (int64_t)(start_m + row);
    xptr[j] = p.x + src * p.x_stride_m;
  }
  const int xlds0 = (tid >> 4) * XPITCH + xc * 16;  // piece j at xlds0 + j*16*XPITCH

  const int nfr = (N + 31) >> 5;
  const uint8_t* wptr[NFW];
#pragma unroll
  for (int f = 0; f < NFW; ++f) {
    int F = pid_n * (BN / 32) + nw * NFW + f;
    F = F < nfr ? F : nfr - 1;  // fragments past N repeat the last one; their columns are dropped in the epilogue
    wptr[f] = p.w + (int64_t)expert * p.w_stride_e + (int64_t)F * nst * 8192 + lane * 16;
  }

  typename FR::acc_t acc[NFW][MFW];
#pragma unroll
  for (int f = 0; f < NFW; ++f)
#pragma unroll
    for (int j = 0; j < MFW; ++j)
#pragma unroll
      for (int i = 0; i < FR::NACC; ++i) acc[f][j][i] = 0.f;

  u32x4_t xreg[XCH];
  i32x8_t wreg[2][NFW][NS];  // [stage parity][column fragment][K-step]
  i32x8_t xf[2][MFW];        // [K-step parity][row fragment]

  // Loads are unconditional: rows past the last valid row re-read it, k past K re-reads the row's last 16 bytes
  // (the padded weights there are zero), stages past the last one re-read the last stage.
  auto load_x_piece = [&](int j, int s) __attribute__((always_inline)) {
    int k0 = s * KC + xc * 16;
    k0 = k0 < K - 16 ? k0 : K - 16;
    xreg[j] = *reinterpret_cast<const u32x4_t*>(xptr[j] + k0);
  };
  auto store_x_piece = [&](int j, int buf) __attribute__((always_inline)) {
    *reinterpret_cast<u32x4_t*>(lds + buf * XBYTES + xlds0 + j * 16 * XPITCH) = xreg[j];
  };
  // weights of K-step t of column fragment f, stage s, into register set SL
  auto load_w = [&](auto slot_c, int f, int t, int s) __attribute__((always_inline)) {
    constexpr int SL = decltype(slot_c)::value;
    s = s < nst ? s : nst - 1;
    const uint8_t* a = wptr[f] + (int64_t)s * 8192 + t * 2048;
    const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(a);
    const u32x4_t hi = *reinterpret_cast<const u32x4_t*>(a + 1024);
    wreg[SL][f][t] = __builtin_bit_cast(i32x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  auto read_xf = [&](int buf, int t, int j, i32x8_t (&out)[MFW]) __attribute__((always_inline)) {
    const uint8_t* a = lds + buf * XBYTES + (j * FM + lr) * XPITCH + t * 64 + h * 32;
    const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(a);
    const u32x4_t hi = *reinterpret_cast<const u32x4_t*>(a + 16);
    out[j] = __builtin_bit_cast(i32x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  template_int<0> S0;
  template_int<1> S1;

  // One stage.  NJ = row fragments with valid rows; PAR = c & 1 = LDS buffer and weight register set.
  // Ops of step t: NJ reads of step t+1's activation fragments (step 3: the next stage's step 0, after the
  // barrier), in steps 0..2 the staging of the next stage's activations (2 NJ pieces over three steps) and in
  // every step two (fragment, K-step) pairs of the next stage's weights.
  auto stage = [&](auto nj_c, auto par_c, int c) __attribute__((always_inline)) {
    constexpr int NJ = decltype(nj_c)::value;
    constexpr int PAR = decltype(par_c)::value;
    using NXT = template_int<PAR ^ 1>;
    constexpr int NM = NJ * NFW;
    constexpr int NP = 2 * NJ;
    constexpr int PPS = (NP + 2) / 3;          // pieces staged per step during steps 0..2
    constexpr int WPS = (NFW * NS + NS - 1) / NS;  // weight (fragment, K-step) pairs loaded per step
    constexpr int NOPS = NJ + PPS + WPS;
    static_for<0, NS>([&](auto t_c) __attribute__((always_inline)) {
      constexpr int t = decltype(t_c)::value;
      constexpr int cur = t & 1, nxt = cur ^ 1;
      auto op = [&](auto o_c) __attribute__((always_inline)) {
        constexpr int o = decltype(o_c)::value;
        if constexpr (o < NJ) {
          if constexpr (t < NS - 1)
            read_xf(PAR, t + 1, o, xf[nxt]);
          else
            read_xf(PAR ^ 1, 0, o, xf[nxt]);
        } else if constexpr (o < NJ + PPS) {
          constexpr int j = t * PPS + (o - NJ);
          if constexpr (t < NS - 1 && j < NP) {
            store_x_piece(j, PAR ^ 1);
            load_x_piece(j, c + 2);
          }
        } else {
          constexpr int w = t * WPS + (o - NJ - PPS);
          if constexpr (w < NFW * NS) load_w(NXT{}, w % NFW, w / NFW, c + 1);  // in the order the K-steps use them
        }
      };
      static_for<0, NM>([&](auto m_c) __attribute__((always_inline)) {
        constexpr int m = decltype(m_c)::value;
        constexpr int j = m / NFW, f = m % NFW;
        acc[f][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wreg[PAR][f][t], xf[cur][j], acc[f][j], 0, 0, 0, 0, 0, 0);
        if constexpr (t == NS - 1 && m == 0) {
          // every wave has fetched its last operands of this buffer (during step 2) and written its share of
          // the next one (steps 0..2)
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        }
        static_for<(m * NOPS) / NM, ((m + 1) * NOPS) / NM>(op);
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };

  auto run = [&](auto nj_c) __attribute__((always_inline)) {
    constexpr int NJ = decltype(nj_c)::value;
    constexpr int NP = 2 * NJ;
    // Prologue: stage 0 without overlap; the loads left in flight (activations, then weights, of stage 1) are
    // issued in the order the steady state leaves them in at the top of a stage.
    static_for<0, NP>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 0); });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NFW * NS>([&](auto wc) __attribute__((always_inline)) { load_w(S0, decltype(wc)::value % NFW, decltype(wc)::value / NFW, 0); });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NP>([&](auto jc) __attribute__((always_inline)) { store_x_piece(decltype(jc)::value, 0); });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NP>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 1); });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NFW * NS>([&](auto wc) __attribute__((always_inline)) { load_w(S1, decltype(wc)::value % NFW, decltype(wc)::value / NFW, 1); });
    __builtin_amdgcn_sched_barrier(0);
    // the claim issued when the tile started has had the prologue's loads to travel behind
    if (claim_now && pass_off == 0 && tid == 0) next_tile_s[tile_par ^ 1] = claimer.resolve();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) { read_xf(0, 0, decltype(jc)::value, xf[0]); });
    __builtin_amdgcn_sched_barrier(0);
    int c = 0;
    for (; c + 1 < nst; c += 2) {
      stage(nj_c, S0, c);
      stage(nj_c, S1, c + 1);
    }
    if (c < nst) stage(nj_c, S0, c);
  };
  static_for<1, MFW + 1>([&](auto n_c) __attribute__((always_inline)) {
    if (nj == decltype(n_c)::value) run(n_c);
  });
  // (the LDS reads after the last stage's barrier fetch operands of a stage that does not exist and are not
  // used, so the next pass may overwrite the buffers without another barrier)
  gemm_epilogue<FM, 1, MFW, NFW, SWIGLU>(p, acc, expert, off_m, start_m, blk_off + blk_rows, pid_n * BN + nw * NFW * FM,
                                         pid_n * BN + BN <= N, 0, lr, h);
  }  // passes
  // next tile
  if (dyn) {
    // written by thread 0 before this tile's first workgroup barrier; the slot is not written again before the
    // first barrier of the tile after the next, which no wave passes before it has read this value
    tile_par ^= 1;
    pid = claim_now ? __builtin_amdgcn_readfirstlane(next_tile_s[tile_par]) : pid_second;
    ++n_tile;
  } else {
    round0 += (int)gridDim.x;
    const int in_round = live - round0 < (int)gridDim.x ? live - round0 : (int)gridDim.x;
    pid = (int)blockIdx.x < in_round ? round0 + xcd_remap(blockIdx.x, in_round) : -1;
  }
  }  // tiles
  if (dyn) claimer.finish();
}

template <int BLKM, int MFW, int NFW>
int32_t launch_f8n(const GemmParams& p, int grid_m, bool swiglu, hipStream_t st) {
  constexpr int LDS_BYTES = 2 * MFW * 32 * (256 + 16);
  GemmParams q = p;
  q.grid_n = (int)cdiv(p.N, 128 * NFW);
  int64_t grid = (int64_t)grid_m * q.grid_n;
  if (grid <= 0) return TK_OK;
  if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: grid too large");
  q.total_tiles = (int32_t)grid;
  // persistent grid, one workgroup per CU (the register ring and the accumulators take a wave's whole budget)
  const int64_t resident = (int64_t)busy_cu_count(p.idle_cus);
  if (grid > resident) grid = resident;
  auto launch = [&](auto kern) -> int32_t {
    if (const int32_t rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), LDS_BYTES)) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), LDS_BYTES, st, q);
    return check_launch("moe_gemm_f8n_kernel");
  };
  if (swiglu) return launch(moe_gemm_f8n_kernel<BLKM, MFW, NFW, true>);
  return launch(moe_gemm_f8n_kernel<BLKM, MFW, NFW, false>);
}

}  // namespace

int32_t gemm_launch_f8n(const GemmParams& p, int block_m, int grid_m, bool swiglu, hipStream_t st) {
  //                                          BLKM MFW NFW
  if (block_m == 256) return launch_f8n<256, 4, 2>(p, grid_m, swiglu, st);
  return launch_f8n<128, 4, 2>(p, grid_m, swiglu, st);
}

}  // namespace tk
