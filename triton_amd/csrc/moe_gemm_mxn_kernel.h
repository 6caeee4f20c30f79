// The persistent prefill kernel for bf16 activations x tiled MXFP4 weights and its launcher, shared by the translation
// units that instantiate it (moe_gemm_mxn.hip: bf16 output; moe_gemm_mxn_mx.hip: MX-quantised output).
#pragma once
#include "gemm_common.h"

namespace tk {
namespace {

// ------------------------------------------------------------------------------------------------
// MXFP4 weights in the tile-native layout (prefill: block_m 64 / 128)
// ------------------------------------------------------------------------------------------------
// Weight layout (built once per model by the host from the K-contiguous form): per expert, per fragment F of
// 32 output columns, per K-stage s of 128: one 2 KiB block [q:2][lane:64][16 B]; lane = h*32 + lr holds the
// packed e2m1 bytes of column F*32 + lr for k in [s*128 + h*64 + q*32, +32).  Scales: one 128 B block
// [lr:32][4] per (F, s) with the four e8m0 bytes of column lr's stage.  N is padded to 32 and K to 128 with
// zero weights.  A wave owns two column fragments and reads its weights straight from global memory into
// registers (every load instruction fetches 1 KiB contiguous, nothing is shared between waves, so they
// bypass LDS); only the gathered activation rows, which all four waves need, are staged through LDS.
//
// Pipeline per K-stage (8 MFMA steps of k = 16): the MFMAs of step t are interleaved, in program order pinned
// by scheduling barriers, with the LDS reads and e2m1 -> bf16 conversions of step t+1, with the LDS writes of
// the next stage's activations and the global loads of the stage after it.  One workgroup barrier per stage
// sits in step 7, after every wave has fetched its last operands of the current LDS buffer.
//
// G = row groups: with G = 2 the workgroup has eight waves; waves 0-3 own the even 32-row fragments of the tile
// and waves 4-7 the odd ones (same columns), so every SIMD holds two waves whose MFMAs, conversions and memory
// instructions overlap in hardware, while the weights are still fetched from L2 / HBM once per 64*MFW rows.
//
// NFW = column fragments per wave (tile width 128 * NFW): the activation tile is fetched from L2 once per column
// tile, so wider tiles cut the L2 -> L1 traffic, which is what bounds this kernel at prefill shapes.
// WD / XD = depth of the weight register ring (2 or 4) / of the activation staging registers (1 or 2).
// Tail tiles: when at most four of a tile's column fragments lie below N (NFW = 2), wave w multiplies fragment w only
// (its second fragment is loaded but neither converted nor multiplied, and its stores are dropped).
// BLKM = rows of a row block in the ragged metadata (block_m).  A tile processes its block in passes of
// BM = 32 * MFW * G rows; with BLKM = 256 and MFW = 5 an expert of up to 160 rows is ONE tile (weights read
// once, no nearly empty second tile) and only larger blocks take a second pass.

template <int BLKM, int MFW, int NFW, int G, int WD, int XD, bool SWIGLU, bool MXOUT>
__global__ __launch_bounds__(256 * G) void moe_gemm_mxn_kernel(const GemmParams p) {
  static_assert(!MXOUT || G == 1, "the MX-output epilogue is written for one row group");
  typedef Frag<32> FR;
  constexpr int FM = 32, NT = 256 * G, BM = MFW * 32 * G, BN = 128 * NFW, KC = 128;
  static_assert((WD == 2 || WD == 4) && (XD == 1 || XD == 2), "ring depths");
  static_assert(BM <= NT && BN <= NT, "one thread per tile row and per tile column fetches the epilogue operands");
  constexpr int XPITCH = KC * 2 + 16;
  constexpr int XBYTES = BM * XPITCH;
  constexpr int XCH = BM * 16 / NT;  // 16-byte activation pieces per thread per stage (4 or 8)
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ int32_t soffs_s[kMetaSlices], ssize_s[kMetaSlices], boffs_s[kMetaSlices + 1];
  // per-unit operands, two sets used in turn: set (u & 1) holds unit u's epilogue operands and unit u+1's gather indices
  __shared__ __attribute__((aligned(16))) float bias_s[2][BN];
  __shared__ float gam_s[2][BM];
  __shared__ int32_t dst_s[2][BM], gidx_s[2][BM];
  __shared__ int next_tile_s[2];  // slot (n & 1): id of the tile after the next, written during this workgroup's n-th tile

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nw = wave & 3, grp = wave >> 2;  // column quarter, row group
  const int lr = lane & 31, h = lane >> 5;
  const int K = p.K, N = p.N;
  const int nst = p.w_nst;
  const int nfr = (N + 31) >> 5;
  const int xc = tid & 15;
  const int xlds0 = (tid >> 4) * XPITCH + xc * 16;  // activation piece j at xlds0 + j*(NT/16)*XPITCH
  const int grid = (int)gridDim.x;
  const bool ragged = p.slice_sizes != nullptr;
  const int nblk = ragged ? p.block_offs[p.n_slices] : 0;
  const int live = ragged ? nblk * p.grid_n : p.total_tiles;
  if (ragged) {  // (the host admits at most kMetaSlices slices)
    for (int i = tid; i < p.n_slices; i += NT) {
      soffs_s[i] = p.slice_offs[i];
      ssize_s[i] = p.slice_sizes[i];
      boffs_s[i] = p.block_offs[i];
    }
    if (tid == 0) boffs_s[p.n_slices] = nblk;
  }
  const __amdgpu_buffer_rsrc_t yrsrc = __builtin_amdgcn_make_buffer_rsrc(p.y, 0, p.y_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t ysrsrc = __builtin_amdgcn_make_buffer_rsrc(p.y_mx_scale, 0, MXOUT ? 0x7FFFFFFF : 0, 0x00020000);

  // A unit of work = one pass of BM rows over one tile (a row block of one expert x BN columns).  Persistent
  // workgroups walk over tiles either by a static schedule (round r: tile r * grid + remap(block)) or by claiming them
  // (TileClaimer); either way the ids of the next two tiles are known when a tile ends, so that a unit's gather
  // indices and epilogue operands are fetched two and one unit ahead, and its first loads are issued before the
  // previous unit's epilogue arithmetic.
  struct Unit {
    int expert, blk_off, blk_rows, pid_n, start_m, pass_off;
    bool valid;
    bool tail;  // at most four column fragments of the tile lie below N: one per wave (NFW = 2)
  };
  auto tile_unit = [&](int pid) __attribute__((always_inline)) -> Unit {
    Unit u;
    int eM;
    if (ragged) {
      // Tiles are ordered (expert, column tile, row block): the row blocks of one expert that share a column
      // tile get consecutive ids, run at the same time on one XCD and stream the same weights through its L2.
      // The expert is the last slice whose first block is not past block pid / grid_n (empty slices share an
      // offset with their successor): a binary search in the block offsets kept in LDS.
      const int blk = pid / p.grid_n;
      int lo = 0, hi = p.n_slices;
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (boffs_s[mid] <= blk) lo = mid; else hi = mid;
      }
      u.expert = lo;
      const int first = boffs_s[lo];
      const int nb = boffs_s[lo + 1] - first;
      const int local = pid - first * p.grid_n;
      u.pid_n = local / nb;
      u.blk_off = (local - u.pid_n * nb) * BLKM;
      u.start_m = soffs_s[lo];
      eM = ssize_s[lo];
    } else {
      u.pid_n = pid % p.grid_n;
      u.expert = 0;
      u.blk_off = (pid / p.grid_n) * BLKM;
      u.start_m = 0;
      eM = p.M;
    }
    u.blk_rows = (eM - u.blk_off) < BLKM ? (eM - u.blk_off) : BLKM;
    u.pass_off = 0;
    u.valid = true;
    u.expert = __builtin_amdgcn_readfirstlane(u.expert);
    u.blk_off = __builtin_amdgcn_readfirstlane(u.blk_off);
    u.blk_rows = __builtin_amdgcn_readfirstlane(u.blk_rows);
    u.pid_n = __builtin_amdgcn_readfirstlane(u.pid_n);
    u.start_m = __builtin_amdgcn_readfirstlane(u.start_m);
    u.tail = !MXOUT && NFW == 2 && nfr - u.pid_n * (BN / 32) <= 4;
    return u;
  };
  // the unit after `u`: its next pass, or the first pass of tile `pid_after` (-1: none)
  auto advance = [&](const Unit& u, int pid_after) __attribute__((always_inline)) -> Unit {
    Unit n = u;
    if (u.pass_off + BM < u.blk_rows) {
      n.pass_off = u.pass_off + BM;
    } else if (pid_after >= 0) {
      n = tile_unit(pid_after);
    } else {
      n.valid = false;
    }
    return n;
  };

  // (with the same number of tiles for every workgroup the static schedule is already even, and measured faster)
  // (claiming also needs at least one workgroup per queue, i.e. a grid of 8 or more: a queue's tiles are reached
  // through the workgroups that start on it)
  const bool dyn = p.tile_counters != nullptr && live % grid != 0 && grid >= 8;
  TileClaimer claimer;
  int round0 = 0;
  int pid, pid_next;  // this workgroup's current and next tile id (-1 = none)
  if (dyn) {
    pid = claimer.init(p.tile_counters, live);
    pid_next = pid >= 0 ? claimer.second() : -1;
  } else {
    const int in0 = live < grid ? live : grid;
    pid = (int)blockIdx.x < in0 ? xcd_remap(blockIdx.x, in0) : -1;
    round0 = grid;
    const int in1 = live - round0 < grid ? live - round0 : grid;
    pid_next = (pid >= 0 && (int)blockIdx.x < in1) ? round0 + xcd_remap(blockIdx.x, in1) : -1;
  }
  int n_tile = 0;  // tiles this workgroup has finished
  if (ragged) __syncthreads();

  // ---- per-unit operand addresses: a uniform 64-bit base (scalar registers) plus a 32-bit byte offset per lane, so
  // that they cost one vector register per activation piece and none per weight fragment ----
  uint32_t xoff[XCH];           // byte offset of this thread's row j in x (x spans less than 4 GiB, checked by the host)
  const uint8_t* wbase[NFW];    // uniform: first K-stage of this wave's column fragment f
  const uint8_t* sbase[NFW];
  const uint32_t lane16 = lane * 16, lr4 = lr * 4;
  // gather index (source row of x) of tile row `tid` of unit u, rows past the block's end repeat its last row
  auto unit_gather_index = [&](const Unit& u) __attribute__((always_inline)) -> int {
    int row = u.blk_off + u.pass_off + tid;
    row = row < u.blk_off + u.blk_rows ? row : u.blk_off + u.blk_rows - 1;
    const int srow = u.start_m + row;
    return p.gather ? p.gather[srow] : srow;
  };
  // addresses of unit u from the gather indices staged in gidx_s[set]
  auto unit_pointers = [&](const Unit& u, int set) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < XCH; ++j) {
      const int r = (tid >> 4) + (NT / 16) * j;
      xoff[j] = (uint32_t)gidx_s[set][r] * (uint32_t)(p.x_stride_m * 2);  // the k offset (incl. this thread's chunk) is added per stage
    }
#pragma unroll
    for (int f = 0; f < NFW; ++f) {
      // (tail tiles: fragment nw of the tile is this wave's first, its second lies past N)
      int F = u.pid_n * (BN / 32) + (u.tail ? nw + 4 * f : nw * NFW + f);
      F = F < nfr ? F : nfr - 1;  // fragments past N repeat the last one; their columns are dropped in the epilogue
      wbase[f] = p.w + (int64_t)u.expert * p.w_stride_e + (int64_t)F * nst * 2048;
      sbase[f] = p.w_scale + (int64_t)u.expert * p.ws_stride_e + (int64_t)F * nst * 128;
    }
  };
  // Epilogue operands of a unit as thread `tid` fetches them: bias of tile column tid, gate weight and scatter index of
  // tile row tid.  `unit_operands` only issues the loads and keeps the raw bits (anything computed from a loaded value
  // would make the wave wait for it on the spot); `stage_operands` converts them when they go to LDS, a K loop later.
  uint32_t bias_raw = 0, gam_raw = 0;
  int dst_raw = 0, gidx_v = 0;
  auto unit_operands = [&](const Unit& u) __attribute__((always_inline)) {
    const int off_m = u.blk_off + u.pass_off, blk_end = u.blk_off + u.blk_rows;
    if (p.bias) {
      int n = u.pid_n * BN + (tid < BN ? tid : BN - 1);
      n = n < N ? n : N - 1;
      const int64_t i = (int64_t)u.expert * p.bias_stride_e + n;
      bias_raw = p.bias_is_f32 ? static_cast<const uint32_t*>(p.bias)[i] : (uint32_t)static_cast<const uint16_t*>(p.bias)[i];
    }
    int row = off_m + (tid < BM ? tid : BM - 1);
    row = row < blk_end ? row : blk_end - 1;
    const int srow = u.start_m + row;  // row in expert-sorted order
    if (p.gammas) gam_raw = p.gammas_is_f32 ? static_cast<const uint32_t*>(p.gammas)[srow] : (uint32_t)static_cast<const uint16_t*>(p.gammas)[srow];
    if (p.scatter) dst_raw = p.scatter[srow < p.scatter_len ? srow : p.scatter_len - 1];
  };
  auto stage_operands = [&](const Unit& u, int set) __attribute__((always_inline)) {
    // (the index is made opaque so that the LDS addresses are recomputed here instead of being kept in registers)
    int t = tid;
    asm volatile("" : "+v"(t));
    if (t < BN) bias_s[set][t] = p.bias ? bits_f32(p.bias_is_f32 ? bias_raw : bias_raw << 16) : 0.f;
    if (t < BM) {
      const int off_m = u.blk_off + u.pass_off, blk_end = u.blk_off + u.blk_rows;
      const bool ok = off_m + t < blk_end;
      const int srow = u.start_m + off_m + t;
      int dst = srow;
      if (p.scatter) dst = srow < p.scatter_len ? dst_raw : -1;
      gam_s[set][t] = p.gammas ? bits_f32(p.gammas_is_f32 ? gam_raw : gam_raw << 16) : 1.0f;
      dst_s[set][t] = ok ? dst : -1;
      gidx_s[set][t] = gidx_v;
    }
  };

  typename FR::acc_t acc[NFW][MFW];
  // activation staging registers, XD stages deep: stage c writes X(c+1) from slot (c+1) % XD to LDS and refills it
  // with X(c+1+XD).  (Native vectors: arrays of the HIP uint4 struct were left in scratch memory here.)
  u32x4_t xreg[XD][XCH];
  // weight register ring: stage c uses slot c % WD, loads run WD-1 stages ahead
  u32x4_t wraw[WD][NFW][2];
  uint32_t sd[WD][NFW];
  bf16x8_t xf[2][MFW];
  bf16x8_t wf[2][NFW];

  // Loads are unconditional (no divergent control flow inside the pipeline): rows past the tile's last
  // valid row re-read that row, k past K re-reads the row's last 8 values (the padded weights there are
  // zero), stages past the last one re-read the last stage.
  auto load_x_piece = [&](int j, int s, int slot) __attribute__((always_inline)) {
    int k0 = s * KC + xc * 8;
    k0 = k0 < K - 8 ? k0 : K - 8;
    xreg[slot][j] = *reinterpret_cast<const u32x4_t*>(p.x + (xoff[j] + (uint32_t)(k0 * 2)));
  };
  auto store_x_piece = [&](int j, int buf, int slot) __attribute__((always_inline)) {
    *reinterpret_cast<u32x4_t*>(lds + buf * XBYTES + xlds0 + j * (NT / 16) * XPITCH) = xreg[slot][j];
  };
  auto load_w = [&](auto par_c, int s) __attribute__((always_inline)) {
    constexpr int PAR = decltype(par_c)::value;
    s = s < nst ? s : nst - 1;
#pragma unroll
    for (int f = 0; f < NFW; ++f) {
      wraw[PAR][f][0] = *reinterpret_cast<const u32x4_t*>(wbase[f] + (int64_t)s * 2048 + lane16);
      wraw[PAR][f][1] = *reinterpret_cast<const u32x4_t*>(wbase[f] + (int64_t)s * 2048 + 1024 + lane16);
      sd[PAR][f] = *reinterpret_cast<const uint32_t*>(sbase[f] + (int64_t)s * 128 + lr4);
    }
  };
  // operands of step t of the stage held in LDS buffer `buf` / weight registers PAR
  auto read_xf = [&](int buf, int t, int j, bf16x8_t (&out)[MFW]) __attribute__((always_inline)) {
    out[j] = *reinterpret_cast<const bf16x8_t*>(lds + buf * XBYTES + ((j * G + grp) * FM + lr) * XPITCH + h * 128 + t * 16);
  };
  // The empty volatile asm statements pin the conversion between the MFMAs of its slot: without them the
  // (side-effect free) conversions drift to the start of the next step and serialise with the MFMAs.
  auto make_wf = [&](auto par_c, int t, int f, bf16x8_t (&out)[NFW]) __attribute__((always_inline)) {
    constexpr int PAR = decltype(par_c)::value;
    const u32x4_t v = wraw[PAR][f][t >> 2];
    uint32_t raw = (t & 3) == 0 ? v.x : (t & 3) == 1 ? v.y : (t & 3) == 2 ? v.z : v.w;
    asm volatile("" : "+v"(raw));
    const uint32_t sbyte = (sd[PAR][f] >> (8 * (t >> 2))) >> (16 * h);  // MX block h*2 + t/4 of the stage
    u32x4_t r = __builtin_bit_cast(u32x4_t, dequant8(raw, bits_f32((sbyte & 0xFFu) << 23)));
    asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w));
    out[f] = __builtin_bit_cast(bf16x8_t, r);
  };

  template_int<0> S0;
  template_int<1> S1;
  template_int<2> S2;
  template_int<3> S3;

  // One K-stage.  NJ = row fragments with valid rows (compile-time so the MFMA list is straight-line code);
  // only the 2*NJ activation pieces per thread that cover those fragments are staged.  WS = weight ring slot
  // of this stage (= c % WD); the activation LDS buffer is WS & 1.
  auto stage = [&](auto nj_c, auto gi_c, auto nf_c, auto ws_c, int c) __attribute__((always_inline)) {
    constexpr int NJ = decltype(nj_c)::value;
    constexpr int NFV = decltype(nf_c)::value;  // column fragments of this wave that are multiplied (the loads always cover NFW)
    constexpr int WS4 = decltype(ws_c)::value;  // c % 4
    constexpr int PAR = WS4 & 1;
    using WSC = template_int<WS4 % WD>;                // this stage's weights
    using WSN = template_int<(WS4 + 1) % WD>;          // next stage's weights
    using WSL = template_int<(WS4 + WD - 1) % WD>;     // slot to refill: stage c + WD - 1
    constexpr int XS = (WS4 + 1) % XD;                 // activation register slot holding X(c+1)
    constexpr int WLOAD_STEP = WD == 2 ? 0 : 4;        // the refilled slot was last read in step 6 of stage c-1
    constexpr int GI = decltype(gi_c)::value;  // this wave's row group
    constexpr int NM = NJ * NFV;
    // pieces to stage: a piece covers 16 rows (G = 1) or 32 rows (G = 2); with G = 2 the tile has 2*NJ - 1 or 2*NJ
    // (group 0), 2*NJ or 2*NJ + 1 (group 1) fragments with valid rows, and the larger count is staged
    constexpr int NP = G == 1 ? 2 * NJ : (2 * NJ + GI < XCH ? 2 * NJ + GI : XCH);
    constexpr int PPS = (NP + 3) / 4;    // per step, during steps 0..3
    constexpr int NOPS = NJ + NFV + 4;   // NJ LDS reads, NFV conversions, three staging slots, the weight loads
    static_for<0, 8>([&](auto t_c) __attribute__((always_inline)) {
      constexpr int t = decltype(t_c)::value;
      constexpr int cur = t & 1, nxt = cur ^ 1;
      auto op = [&](auto o_c) __attribute__((always_inline)) {
        constexpr int o = decltype(o_c)::value;
        if constexpr (o == NJ + NFV + 3) {
          if constexpr (t == WLOAD_STEP) load_w(WSL{}, c + WD - 1);
        } else if constexpr (t < 7) {
          if constexpr (o < NJ) {
            read_xf(PAR, t + 1, o, xf[nxt]);
          } else if constexpr (o < NJ + NFV) {
            make_wf(WSC{}, t + 1, o - NJ, wf[nxt]);
          } else if constexpr (t < 4) {
            // next stage's activations: registers -> LDS, then refill the registers for a later stage
            constexpr int half = o - NJ - NFV;
            constexpr int j = t * PPS + half;
            if constexpr (half < PPS && j < NP) {
              store_x_piece(j, PAR ^ 1, XS);
              load_x_piece(j, c + 1 + XD, XS);
            }
          }
        } else {
          if constexpr (o < NJ) {
            read_xf(PAR ^ 1, 0, o, xf[nxt]);
          } else if constexpr (o < NJ + NFV) {
            make_wf(WSN{}, 0, o - NJ, wf[nxt]);
          }
        }
      };
      if constexpr (NM == 0) {
        // a wave without valid rows still stages its share of the activations and joins the barriers
        if constexpr (t == 7) {
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        }
        static_for<0, NOPS>(op);
        __builtin_amdgcn_sched_barrier(0);
      }
      static_for<0, NM>([&](auto m_c) __attribute__((always_inline)) {
        constexpr int m = decltype(m_c)::value;
        constexpr int j = m / NFV, f = m % NFV;
        acc[f][j] = FR::mma(wf[cur][f], xf[cur][j], acc[f][j]);
        if constexpr (t == 7 && m == 0) {
          // every wave has fetched its last operands of this buffer (during step 6) and written its share
          // of the next one (steps 0..3)
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        }
        // ops are dealt as evenly as possible: slot m runs ops [m*NOPS/NM, (m+1)*NOPS/NM)
        static_for<(m * NOPS) / (NM ? NM : 1), ((m + 1) * NOPS) / (NM ? NM : 1)>(op);
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };

  // Stage 0 of a unit (activations of every piece, weights): issued before the previous unit's epilogue arithmetic.
  auto first_loads = [&]() __attribute__((always_inline)) {
    static_for<0, XCH>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 0, 0); });
    __builtin_amdgcn_sched_barrier(0);
    load_w(S0, 0);
    __builtin_amdgcn_sched_barrier(0);
  };

  int up = 0;             // operand set of the current unit
  Unit cur_unit;          // the unit being computed
  int resolve_slot = -1;  // thread 0 writes the claimed tile id into next_tile_s[resolve_slot] before the first barrier
  auto run = [&](auto nj_c, auto gi_c, auto nf_c) __attribute__((always_inline)) {
    constexpr int NJ = decltype(nj_c)::value;
    constexpr int GI = decltype(gi_c)::value;
    constexpr int NFV = decltype(nf_c)::value;
    constexpr int NP = G == 1 ? 2 * NJ : (2 * NJ + GI < XCH ? 2 * NJ + GI : XCH);
    // Prologue: finish stage 0 (its loads were issued by first_loads before the previous unit's epilogue).  The order
    // of the loads left in flight (activations, then weights, of stage 1, then of stage 2) is pinned to the order the
    // steady state leaves them in at the top of a stage: the compiler's wait counts at the loop header are the merge
    // of both paths, and any mismatch makes every iteration wait for the loads it has just issued.
    static_for<0, NP>([&](auto jc) __attribute__((always_inline)) { store_x_piece(decltype(jc)::value, 0, 0); });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NP>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 1, 1 % XD); });
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (WD == 4) {
      load_w(S1, 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (XD == 2) {
      static_for<0, NP>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 2, 0); });
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (WD == 4) {
      load_w(S2, 2);
      __builtin_amdgcn_sched_barrier(0);
    }
    // what was fetched during the previous unit's epilogue goes to LDS: this unit's epilogue operands and the next
    // unit's gather indices (set `up`; its last readers were the epilogue and the address set-up two units back)
    stage_operands(cur_unit, up);
    // the claim issued before the previous epilogue has had that long to travel
    if (resolve_slot >= 0 && tid == 0) next_tile_s[resolve_slot] = claimer.resolve();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) { read_xf(0, 0, decltype(jc)::value, xf[0]); });
    static_for<0, NFV>([&](auto fc) __attribute__((always_inline)) { make_wf(S0, 0, decltype(fc)::value, wf[0]); });
    __builtin_amdgcn_sched_barrier(0);
    // all stages of a group always run inside the loop: a path that skips some and returns to the loop header
    // would again make the header's wait counts cover the loads just issued
    int c = 0;
    for (; c + 3 < nst; c += 4) {
      stage(nj_c, gi_c, nf_c, S0, c);
      stage(nj_c, gi_c, nf_c, S1, c + 1);
      stage(nj_c, gi_c, nf_c, S2, c + 2);
      stage(nj_c, gi_c, nf_c, S3, c + 3);
    }
    if (c < nst) stage(nj_c, gi_c, nf_c, S0, c);
    if (c + 1 < nst) stage(nj_c, gi_c, nf_c, S1, c + 1);
    if (c + 2 < nst) stage(nj_c, gi_c, nf_c, S2, c + 2);
  };
  auto dispatch = [&](auto gi_c, auto nf_c, int nj) __attribute__((always_inline)) {
    constexpr int GI = decltype(gi_c)::value;
    if constexpr (GI == 1) {
      if (nj == 0) {
        run(template_int<0>{}, gi_c, nf_c);
        return;
      }
    }
    static_for<1, MFW + 1>([&](auto n_c) __attribute__((always_inline)) {
      if (nj == decltype(n_c)::value) run(n_c, gi_c, nf_c);
    });
  };
  // (tail tiles multiply one fragment per wave)
  auto dispatch_nf = [&](auto gi_c, bool tail, int nj) __attribute__((always_inline)) {
    if constexpr (NFW == 2) {
      if (tail) {
        dispatch(gi_c, template_int<1>{}, nj);
        return;
      }
    }
    dispatch(gi_c, template_int<NFW>{}, nj);
  };

  if (pid >= 0) {
    Unit& cur = cur_unit;
    cur = tile_unit(pid);
    Unit nxt = advance(cur, pid_next);
    // the first unit has nothing to hide behind: gather indices, addresses, operands, first loads
    if (tid < BM) gidx_s[1][tid] = unit_gather_index(cur);
    __syncthreads();
    unit_pointers(cur, 1);
    unit_operands(cur);
    if (nxt.valid && tid < BM) gidx_v = unit_gather_index(nxt);
    if (dyn && pid_next >= 0) {
      claimer.issue();  // the tile after the next
      resolve_slot = 0;
    }
    first_loads();
    for (;;) {
#pragma unroll
      for (int f = 0; f < NFW; ++f)
#pragma unroll
        for (int j = 0; j < MFW; ++j)
#pragma unroll
          for (int i = 0; i < FR::NACC; ++i) acc[f][j][i] = 0.f;
      const int rows = (cur.blk_rows - cur.pass_off) < BM ? (cur.blk_rows - cur.pass_off) : BM;
      const int nfrag_m = (rows + FM - 1) / FM;  // row fragments that hold valid rows (1..MFW*G)
      const int nj = (nfrag_m - grp + G - 1) / G;  // those of this wave: tile fragments grp, grp + G, ...
      if constexpr (G == 2) {
        if (grp == 1)
          dispatch_nf(template_int<1>{}, cur.tail, nj);
        else
          dispatch_nf(template_int<0>{}, cur.tail, nj);
      } else {
        dispatch_nf(template_int<0>{}, cur.tail, nj);
      }
      resolve_slot = -1;

      // ---- before this unit's epilogue: everything the next units need from memory ----
      const int wcol = cur.tail ? nw * FM : nw * NFW * FM;  // this wave's first column in the tile
      const int ncol0 = cur.pid_n * BN + wcol;
      const bool cur_tail = cur.tail;
      Unit nxt2 = nxt;
      if (nxt.valid) {
        if (cur.pass_off + BM >= cur.blk_rows) {
          // the next unit opens a new tile; the tile after it was claimed during this tile's first prologue (or
          // follows statically)
          pid = pid_next;
          ++n_tile;
          if (dyn) {
            pid_next = __builtin_amdgcn_readfirstlane(next_tile_s[(n_tile - 1) & 1]);
          } else {
            round0 += grid;
            const int in_round = live - round0 < grid ? live - round0 : grid;
            pid_next = (int)blockIdx.x < in_round ? round0 + xcd_remap(blockIdx.x, in_round) : -1;
          }
          if (dyn && pid_next >= 0) {
            claimer.issue();
            resolve_slot = n_tile & 1;
          }
        }
        nxt2 = advance(nxt, pid_next);
        // (these loads and the claim come BEFORE the next unit's first loads: the number of them in flight differs
        // from path to path, and only what is issued after a load makes the wait for that load inexact)
        unit_operands(nxt);
        if (nxt2.valid && tid < BM) gidx_v = unit_gather_index(nxt2);
        __builtin_amdgcn_sched_barrier(0);
        unit_pointers(nxt, up);
        first_loads();
      }
      if constexpr (MXOUT) {
        // (partly filled column tiles are not split among the waves here: a wave's two fragments are one MX block with swiglu)
        staged_mx_epilogue<MFW, NFW, SWIGLU>(p, acc, yrsrc, ysrsrc, bias_s[up], gam_s[up], dst_s[up], wcol, ncol0, lr, h);
      } else if (NFW == 2 && cur_tail) {
        staged_epilogue<G, MFW, NFW, 1, SWIGLU>(p, acc, yrsrc, bias_s[up], gam_s[up], dst_s[up], wcol, ncol0, grp, lr, h);
      } else {
        staged_epilogue<G, MFW, NFW, NFW, SWIGLU>(p, acc, yrsrc, bias_s[up], gam_s[up], dst_s[up], wcol, ncol0, grp, lr, h);
      }
      if (!nxt.valid) break;
      cur = nxt;
      nxt = nxt2;
      up ^= 1;
    }
  }
  if (dyn) claimer.finish();
  if constexpr (!SWIGLU && !MXOUT) {
    if (p.combine_k > 0 && p.tile_counters != nullptr) fused_prefill_combine<NT>(p, tid, grid);
  }
}

template <int BLKM, int MFW, int NFW, int G, int WD, int XD, bool MXOUT>
int32_t launch_mxn(const GemmParams& p, int grid_m, bool swiglu, hipStream_t st) {
  constexpr int LDS_BYTES = 2 * MFW * 32 * G * (128 * 2 + 16);
  GemmParams q = p;
  q.grid_n = (int)cdiv(p.N, 128 * NFW);
  int64_t grid = (int64_t)grid_m * q.grid_n;
  if (grid <= 0) return TK_OK;
  if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: grid too large");
  q.total_tiles = (int32_t)grid;
  // persistent grid: one workgroup per CU (a wave's registers leave no room for a second one on its SIMD)
  const int64_t resident = (int64_t)busy_cu_count(p.idle_cus);
  if (grid > resident) grid = resident;
  auto launch = [&](auto kern) -> int32_t {
    if (const int32_t rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), LDS_BYTES)) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256 * G), LDS_BYTES, st, q);
    return check_launch("moe_gemm_mxn_kernel");
  };
  if (swiglu) return launch(moe_gemm_mxn_kernel<BLKM, MFW, NFW, G, WD, XD, true, MXOUT>);
  return launch(moe_gemm_mxn_kernel<BLKM, MFW, NFW, G, WD, XD, false, MXOUT>);
}

}  // namespace
}  // namespace tk
