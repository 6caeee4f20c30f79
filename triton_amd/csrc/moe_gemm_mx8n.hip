#include "gemm_common.h"

namespace tk {
namespace {

// ------------------------------------------------------------------------------------------------
// MXFP8 activations x MXFP4 weights in the tile-native layout (prefill): scaled MFMA, no conversion anywhere
// ------------------------------------------------------------------------------------------------
// Both operands stay in their storage formats down to the matrix core: v_mfma_scale_f32_32x32x64_f8f6f4 takes the
// packed e2m1 weights (A operand, format fp4), the e4m3 activations (B operand) and one e8m0 scale byte per lane for
// each, and multiplies both block scales in.  A lane of half h supplies 32 consecutive k of its column / row to one
// instruction, which is exactly one MX block, so the tiled weight layout of the bf16-activation kernel serves as
// it is: piece q of a lane holds k in [s*128 + h*64 + q*32, +32) and byte 2h + q of the stage's scale dword is that
// block's scale (the dword is shifted by 16h once per stage, the instruction's op_sel picks byte q).  The
// activation rows (gathered, one byte per element, 128 bytes per row and stage) are staged through LDS with their
// four e8m0 bytes of the stage in the row's pad.  With a 4-bit and an 8-bit operand the instruction does not pair a
// lane's 32 values one to one: the 8-bit lane of half h holds k' = 16h..16h+15 and 32+16h..32+16h+15 of the
// instruction's 64, while its scale byte still covers k' in [32h, 32h+32), so a lane reads 16 bytes of each of the
// step's two MX blocks (measured with a one-hot probe; exact against a float64 model with random data and scales).
// A K-stage is two MFMA steps (q = 0, 1); structure as in the FP8 kernel: four waves, each owning NFW column
// fragments whose weights go global memory -> register double buffer -> MFMA, all sharing the row fragments of the
// tile through an LDS double buffer; persistent grid, (expert, column tile, row block) tile order.
//
// MXOUT: the output is MX-quantised along N from the fp32 accumulators (after bias, activation and gate weight):
// blocks of 32 output columns, one e8m0 scale byte per block (round-up rule) to y_mx_scale, e4m3 values to y.  A
// wave's 64 accumulator columns are one block with swiglu (two without), half of it in each lane half.
template <int MFW, int NFW, bool SWIGLU>
__device__ __forceinline__ void mx_out_epilogue(const GemmParams& p, f32x16_t (&acc)[NFW][MFW], int expert, int off_m, int start_m, int eM,
                                                int ncol0, int lr, int h) {
  const int N = p.N;
  const int NOUT = SWIGLU ? N / 2 : N;
  const float nalpha_log2e = -p.alpha * 1.4426950408889634f;
  const float limit = p.has_limit ? p.limit : INFINITY;
  uint8_t* yb = reinterpret_cast<uint8_t*>(p.y);
  // everything rows and columns need from memory is fetched before the arithmetic starts: per-row gate weight and
  // destination (rows past the slice read its last row), per-column bias (4 consecutive columns per register group)
  float gam[MFW];
  int64_t dst[MFW];
  bool ok[MFW];
#pragma unroll
  for (int j = 0; j < MFW; ++j) {
    const int row = off_m + j * 32 + lr;  // row inside the slice
    ok[j] = row < eM;
    const int srow = start_m + (ok[j] ? row : eM - 1);
    gam[j] = p.gammas ? load_scalar(p.gammas, srow, p.gammas_is_f32) : 1.0f;
    dst[j] = srow;
    if (p.scatter) {
      const int sr = srow < p.scatter_len ? srow : p.scatter_len - 1;
      const int v = p.scatter[sr];
      dst[j] = srow < p.scatter_len ? v : -1;
    }
  }
  float b4[NFW][4][4];  // [fragment][register group q][i]: bias of column ncol0 + f*32 + 8q + 4h + i
#pragma unroll
  for (int f = 0; f < NFW; ++f)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n0 = ncol0 + f * 32 + 8 * q + 4 * h;
      const int64_t bo = (int64_t)expert * p.bias_stride_e + n0;
      if (!p.bias) {
#pragma unroll
        for (int i = 0; i < 4; ++i) b4[f][q][i] = 0.f;
      } else if (n0 + 4 <= N && p.bias_vec) {
        if (p.bias_is_f32) {
          const float4 t = *reinterpret_cast<const float4*>(static_cast<const float*>(p.bias) + bo);
          b4[f][q][0] = t.x, b4[f][q][1] = t.y, b4[f][q][2] = t.z, b4[f][q][3] = t.w;
        } else {
          const uint2 t = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(p.bias) + bo);
          b4[f][q][0] = bits_f32(t.x << 16), b4[f][q][1] = bits_f32(t.x & 0xFFFF0000u);
          b4[f][q][2] = bits_f32(t.y << 16), b4[f][q][3] = bits_f32(t.y & 0xFFFF0000u);
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) b4[f][q][i] = n0 + i < N ? load_scalar(p.bias, bo + i, p.bias_is_f32) : 0.f;
      }
    }
#pragma unroll
  for (int j = 0; j < MFW; ++j) {
    const bool okj = ok[j] && dst[j] >= 0;
    const float g = gam[j];
    // values of this lane: o[f][u][i]; with swiglu 4 outputs per (f, u) at output column (ncol0 + f*32 + 16u + 8h)/2 + i,
    // without 8 outputs at column ncol0 + f*32 + 16u + 8h + i
    constexpr int VO = SWIGLU ? 4 : 8;
    float o[NFW][2][VO];
#pragma unroll
    for (int f = 0; f < NFW; ++f)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // registers 8u..8u+3 hold columns 16u + 4h + i, registers 8u+4..8u+7 columns 16u + 8 + 4h + i; after the two
          // lane halves exchange their 4-column groups a lane holds 8 consecutive columns from 16u + 8h
          const float a_lo = acc[f][j][8 * u + i] + b4[f][2 * u][i], a_hi = acc[f][j][8 * u + 4 + i] + b4[f][2 * u + 1][i];
          auto sw = __builtin_amdgcn_permlane32_swap(f32_bits(a_lo), f32_bits(a_hi), false, false);
          v[i] = bits_f32(sw[0]);
          v[4 + i] = bits_f32(sw[1]);
        }
#pragma unroll
        for (int i = 0; i < VO; ++i) o[f][u][i] = SWIGLU ? swiglu_f(v[2 * i], v[2 * i + 1], nalpha_log2e, limit) * g : v[i] * g;
      }
    // MX blocks of 32 output columns: with swiglu the wave's 32 outputs of a row (both fragments, both lane halves),
    // without it one block per fragment.  Columns past the end count as zero.
    constexpr int NB = SWIGLU ? 1 : NFW;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      float m = 0.f;
#pragma unroll
      for (int f = 0; f < NFW; ++f) {
        if (!SWIGLU && f != b) continue;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < VO; ++i) {
            const int col = SWIGLU ? (ncol0 + f * 32 + 16 * u + 8 * h) / 2 + i : ncol0 + f * 32 + 16 * u + 8 * h + i;
            const float a = col < NOUT ? fabsf(o[f][u][i]) : 0.f;
            m = a > m ? a : m;  // (a NaN never wins: the block's scale then comes from its finite values)
          }
      }
      const float other = __shfl_xor(m, 32);
      m = other > m ? other : m;
      const uint32_t sbits = mx_scale_bits(m, TK_E4M3, TK_MX_ROUND_UP);
      const float inv = mx_inv_scale(sbits);
      const int blk_col0 = SWIGLU ? ncol0 / 2 : ncol0 + b * 32;  // first output column of the block
      if (okj && h == 0 && blk_col0 < NOUT) p.y_mx_scale[dst[j] * p.ys_stride_m + blk_col0 / 32] = (uint8_t)(sbits >> 23);
#pragma unroll
      for (int f = 0; f < NFW; ++f) {
        if (!SWIGLU && f != b) continue;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int col0 = SWIGLU ? (ncol0 + f * 32 + 16 * u + 8 * h) / 2 : ncol0 + f * 32 + 16 * u + 8 * h;
          float qv[VO];
#pragma unroll
          for (int i = 0; i < VO; ++i) qv[i] = mx_clamp(o[f][u][i] * inv, 448.0f);
          uint8_t* yrow = yb + dst[j] * p.y_stride_m + col0;
          if (okj && col0 + VO <= NOUT && p.y_vec) {
            int w0 = 0;
            w0 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[0], qv[1], w0, false);
            w0 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[2], qv[3], w0, true);
            if constexpr (VO == 8) {
              int w1 = 0;
              w1 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[4], qv[5], w1, false);
              w1 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[6], qv[7], w1, true);
              *reinterpret_cast<uint2*>(yrow) = make_uint2((uint32_t)w0, (uint32_t)w1);
            } else {
              *reinterpret_cast<uint32_t*>(yrow) = (uint32_t)w0;
            }
          } else if (okj) {
#pragma unroll
            for (int i = 0; i < VO; ++i)
              if (col0 + i < NOUT) yrow[i] = (uint8_t)e4m3_byte(qv[i]);
          }
        }
      }
    }
  }
}

template <int BLKM, int MFW, int NFW, bool SWIGLU, bool MXOUT>
__global__ __launch_bounds__(256) void moe_gemm_mx8n_kernel(const GemmParams p) {
  typedef Frag<32> FR;
  constexpr int FM = 32, BM = MFW * 32, BN = 128 * NFW, KC = 128, NS = 2;
  constexpr int XPITCH = KC + 16;  // 128 value bytes, 4 scale bytes, pad
  constexpr int XBYTES = BM * XPITCH;
  constexpr int XCH = BM / 32;  // 16-byte activation pieces per thread per stage (8 pieces per row, 32 rows per sweep)
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int nw = __builtin_amdgcn_readfirstlane(tid >> 6);  // column quarter of the tile
  const int lr = lane & 31, h = lane >> 5;
  const int K = p.K, N = p.N;
  const int nst = p.w_nst;  // stages of 128
  const int grid = (int)gridDim.x;
  const int live = p.slice_sizes ? p.block_offs[p.n_slices] * p.grid_n : p.total_tiles;
  for (int round0 = 0; round0 < live; round0 += grid) {
  const int in_round = live - round0 < grid ? live - round0 : grid;
  if ((int)blockIdx.x >= in_round) break;
  const int pid = round0 + xcd_remap(blockIdx.x, in_round);
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

  // ---- activation staging: piece j of this thread = row 32 j + tid/8, 16-byte chunk tid%8 of the stage; the
  // stage's four scale bytes of row `tid` (tid < BM) travel with them ----
  const int xc = tid & 7;
  const uint8_t* xptr[XCH];
#pragma unroll
  for (int j = 0; j < XCH; ++j) {
    int row = off_m + (tid >> 3) + 32 * j;
    row = row < eM ? row : eM - 1;
    const int64_t src = p.gather ? (int64_t)p.gather[start_m + row] : (int64_t)(start_m + row);
    xptr[j] = p.x + src * p.x_stride_m;
  }
  const uint8_t* xsptr;
  {
    int row = off_m + (tid < BM ? tid : BM - 1);
    row = row < eM ? row : eM - 1;
    const int64_t src = p.gather ? (int64_t)p.gather[start_m + row] : (int64_t)(start_m + row);
    xsptr = p.x_mx_scale + src * p.xs_stride_m;
  }
  const int xlds0 = (tid >> 3) * XPITCH + xc * 16;  // piece j at xlds0 + j*32*XPITCH
  const int kblocks = (K + 31) >> 5;                // scale bytes per activation row (>= 4, checked by the host)

  const int nfr = (N + 31) >> 5;
  const uint8_t* wptr[NFW];
  const uint8_t* sptr[NFW];
#pragma unroll
  for (int f = 0; f < NFW; ++f) {
    int F = pid_n * (BN / 32) + nw * NFW + f;
    F = F < nfr ? F : nfr - 1;  // fragments past N repeat the last one; their columns are dropped in the epilogue
    wptr[f] = p.w + (int64_t)expert * p.w_stride_e + (int64_t)F * nst * 2048 + lane * 16;
    sptr[f] = p.w_scale + (int64_t)expert * p.ws_stride_e + (int64_t)F * nst * 128 + lr * 4;
  }

  typename FR::acc_t acc[NFW][MFW];
#pragma unroll
  for (int f = 0; f < NFW; ++f)
#pragma unroll
    for (int j = 0; j < MFW; ++j)
#pragma unroll
      for (int i = 0; i < FR::NACC; ++i) acc[f][j][i] = 0.f;

  // Register rings: a stage of two MFMA steps is too short to cover a memory round trip, so the weights of stage c + 3
  // and the activations of stage c + 3 are requested while stage c computes (weights: four slots, stage c uses slot
  // c % 4; activations: two slots, slot (c + 1) % 2 holds stage c + 1 until stage c has written it to LDS).
  constexpr int WD = 4, XD = 2;
  u32x4_t xreg[XD][XCH];
  uint32_t xsreg[XD] = {0, 0};
  int xsshift[XD] = {0, 0};   // blocks by which the dword in xsreg starts before block 4 s of its stage
  u32x4_t wraw[WD][NFW][NS];  // [ring slot][column fragment][step]
  uint32_t sd[WD][NFW];       // the stage's four weight scale bytes of this lane's column
  i32x8_t xf[2][MFW];         // [step parity][row fragment]
  uint32_t xs[2][MFW];        // [stage parity]: the stage's activation scale bytes of this lane's rows, this half's two in bytes 0 / 1

  // Loads are unconditional: rows past the last valid row re-read it, k past K re-reads the row's last 16 bytes /
  // last scale bytes (the padded weights there are zero), stages past the last one re-read the last stage.
  auto load_x_piece = [&](int j, int s, int slot) __attribute__((always_inline)) {
    int k0 = s * KC + xc * 16;
    k0 = k0 < K - 16 ? k0 : K - 16;
    xreg[slot][j] = *reinterpret_cast<const u32x4_t*>(xptr[j] + k0);
  };
  auto load_x_scale = [&](int s, int slot) __attribute__((always_inline)) {
    // four scale bytes from block 4 s on (any alignment); a stage that reaches past the row's last block reads the
    // last four blocks instead.  Only the load is issued here: the bytes are moved into place when they go to LDS
    // (anything computed from the loaded value now would make the wave wait for it on the spot).
    int b0 = s * 4;
    b0 = b0 < kblocks - 4 ? b0 : kblocks - 4;
    uint32_t v;
    __builtin_memcpy(&v, xsptr + b0, 4);
    xsreg[slot] = v;
    xsshift[slot] = s * 4 - b0;
  };
  auto store_x_piece = [&](int j, int buf, int slot) __attribute__((always_inline)) {
    *reinterpret_cast<u32x4_t*>(lds + buf * XBYTES + xlds0 + j * 32 * XPITCH) = xreg[slot][j];
  };
  auto store_x_scale = [&](int buf, int slot) __attribute__((always_inline)) {
    // block 4 s of the stage goes to byte 0; blocks past the row's end get the neutral scale 2^0 (their weights are zero)
    const int sh = xsshift[slot] < 4 ? xsshift[slot] : 4;
    const uint64_t wide = ((uint64_t)0x7F7F7F7Fu << 32) | xsreg[slot];
    const uint32_t v = (uint32_t)(wide >> (8 * sh));
    // (no branch inside the K loop: threads past the tile's rows write into the unused pad bytes of a row)
    const int at = tid < BM ? tid * XPITCH + KC : (tid - BM) * XPITCH + KC + 4;
    *reinterpret_cast<uint32_t*>(lds + buf * XBYTES + at) = v;
  };
  auto load_w = [&](auto slot_c, int s) __attribute__((always_inline)) {
    constexpr int SL = decltype(slot_c)::value;
    s = s < nst ? s : nst - 1;
#pragma unroll
    for (int f = 0; f < NFW; ++f) {
      wraw[SL][f][0] = *reinterpret_cast<const u32x4_t*>(wptr[f] + (int64_t)s * 2048);
      wraw[SL][f][1] = *reinterpret_cast<const u32x4_t*>(wptr[f] + (int64_t)s * 2048 + 1024);
      sd[SL][f] = *reinterpret_cast<const uint32_t*>(sptr[f] + (int64_t)s * 128);
    }
  };
  auto read_xf = [&](int buf, int q, int j, i32x8_t (&out)[MFW]) __attribute__((always_inline)) {
    // (the instruction pairs the fp4 operand's nibble i of lane half hh with the 8-bit operand's k = 32 hh + i, which
    // it takes from byte i of half 0 for i < 16 and byte i - 16 of half 1 otherwise, and likewise bytes 16..31 for the
    // second 32: a lane of half h therefore supplies bytes [16 h, 16 h + 16) of both of the step's MX blocks)
    const uint8_t* a = lds + buf * XBYTES + (j * FM + lr) * XPITCH + q * 32 + h * 16;
    const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(a);
    const u32x4_t hi = *reinterpret_cast<const u32x4_t*>(a + 64);
    out[j] = __builtin_bit_cast(i32x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  auto read_xs = [&](int buf, int j, uint32_t (&out)[MFW]) __attribute__((always_inline)) {
    out[j] = *reinterpret_cast<const uint32_t*>(lds + buf * XBYTES + (j * FM + lr) * XPITCH + KC) >> (16 * h);
  };

  template_int<0> S0;
  template_int<1> S1;
  template_int<2> S2;
  template_int<3> S3;

  // One stage.  NJ = row fragments with valid rows; WS4 = c % 4: weight ring slot, its low bit the LDS buffer and the
  // activation scale set.  The MFMAs of step q are interleaved with the LDS reads of the next step's activation
  // fragments (during step 1: the next stage's step 0 and its scale bytes, behind the barrier), and during step 0
  // with the staging of the next stage's activations, the refill of their registers and the weight loads.
  auto stage = [&](auto nj_c, auto ws_c, int c) __attribute__((always_inline)) {
    constexpr int NJ = decltype(nj_c)::value;
    constexpr int WS4 = decltype(ws_c)::value;
    constexpr int PAR = WS4 & 1;
    using WSL = template_int<(WS4 + WD - 1) % WD>;  // slot to refill with stage c + WD - 1 (stage c - 1 used it)
    constexpr int XS = (WS4 + 1) % XD;              // activation register slot holding stage c + 1
    constexpr int NM = NJ * NFW;
    constexpr int NOPS = 2 * NJ + 2;  // NJ reads, NJ staging pieces, the scale staging, the weight loads
    uint32_t sdh[NFW];
#pragma unroll
    for (int f = 0; f < NFW; ++f) sdh[f] = sd[WS4][f] >> (16 * h);
    static_for<0, NS>([&](auto q_c) __attribute__((always_inline)) {
      constexpr int q = decltype(q_c)::value;
      constexpr int cur = q & 1, nxt = cur ^ 1;
      auto op = [&](auto o_c) __attribute__((always_inline)) {
        constexpr int o = decltype(o_c)::value;
        if constexpr (o < NJ) {
          if constexpr (q == 0) {
            read_xf(PAR, 1, o, xf[nxt]);
          } else {
            read_xf(PAR ^ 1, 0, o, xf[nxt]);
            read_xs(PAR ^ 1, o, xs[PAR ^ 1]);
          }
        } else if constexpr (o < 2 * NJ) {
          if constexpr (q == 0) {
            constexpr int j = o - NJ;
            store_x_piece(j, PAR ^ 1, XS);
            load_x_piece(j, c + 1 + XD, XS);
          }
        } else if constexpr (o == 2 * NJ) {
          if constexpr (q == 0) {
            store_x_scale(PAR ^ 1, XS);
            load_x_scale(c + 1 + XD, XS);
          }
        } else {
          if constexpr (q == 0) load_w(WSL{}, c + WD - 1);
        }
      };
      static_for<0, NM>([&](auto m_c) __attribute__((always_inline)) {
        constexpr int m = decltype(m_c)::value;
        constexpr int j = m / NFW, f = m % NFW;
        const u32x4_t wv = wraw[WS4][f][q];
        const i32x8_t a = {(int)wv.x, (int)wv.y, (int)wv.z, (int)wv.w, 0, 0, 0, 0};
        acc[f][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, xf[cur][j], acc[f][j], 4 /* A: e2m1 */, 0 /* B: e4m3 */, q, (int)sdh[f], q,
                                                                     (int)xs[PAR][j]);
        if constexpr (q == NS - 1 && m == 0) {
          // every wave has fetched its last operands of this buffer (during step 0) and written its share of the
          // next one (step 0)
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
    // Prologue: stage 0 without overlap; the loads left in flight (activations, scales, weights of stage 1, then of
    // stage 2) are issued in the order the steady state leaves them in at the top of a stage.
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 0, 0); });
    load_x_scale(0, 0);
    __builtin_amdgcn_sched_barrier(0);
    load_w(S0, 0);
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) { store_x_piece(decltype(jc)::value, 0, 0); });
    store_x_scale(0, 0);
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 1, 1); });
    load_x_scale(1, 1);
    __builtin_amdgcn_sched_barrier(0);
    load_w(S1, 1);
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 2, 0); });
    load_x_scale(2, 0);
    __builtin_amdgcn_sched_barrier(0);
    load_w(S2, 2);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) {
      read_xf(0, 0, decltype(jc)::value, xf[0]);
      read_xs(0, decltype(jc)::value, xs[0]);
    });
    __builtin_amdgcn_sched_barrier(0);
    // all stages of a group always run inside the loop (a path that skips some and returns to the loop header would
    // make the header's wait counts cover the loads just issued)
    int c = 0;
    for (; c + 3 < nst; c += 4) {
      stage(nj_c, S0, c);
      stage(nj_c, S1, c + 1);
      stage(nj_c, S2, c + 2);
      stage(nj_c, S3, c + 3);
    }
    if (c < nst) stage(nj_c, S0, c);
    if (c + 1 < nst) stage(nj_c, S1, c + 1);
    if (c + 2 < nst) stage(nj_c, S2, c + 2);
  };
  static_for<1, MFW + 1>([&](auto n_c) __attribute__((always_inline)) {
    if (nj == decltype(n_c)::value) run(n_c);
  });
  // (the LDS reads after the last stage's barrier fetch operands of a stage that does not exist and are not
  // used, so the next pass may overwrite the buffers without another barrier)
  if constexpr (MXOUT)
    mx_out_epilogue<MFW, NFW, SWIGLU>(p, acc, expert, off_m, start_m, blk_off + blk_rows, pid_n * BN + nw * NFW * FM, lr, h);
  else
    gemm_epilogue<FM, 1, MFW, NFW, SWIGLU>(p, acc, expert, off_m, start_m, blk_off + blk_rows, pid_n * BN + nw * NFW * FM,
                                           pid_n * BN + BN <= N, 0, lr, h);
  }  // passes
  }  // rounds
}

#ifdef TK_MX8_STAMPS
// diagnostic build only: per workgroup, sums of shader-clock cycles spent in [0] the K loops' prologues, [1] the K
// loops, [2] the preparation of the next unit, [3] the epilogues; [4] units, [5] K-stages, [6] whole kernel
__device__ long long mx8_stamps[1024][8];
#define MX8_T() ((long long)__builtin_amdgcn_s_memtime())
#define MX8_ADD(n, v) do { if (threadIdx.x == 0) mx8_stamps[blockIdx.x][n] += (v); } while (0)
#else
#define MX8_T() 0ll
#define MX8_ADD(n, v) do {} while (0)
#endif

// The same K loop inside persistent workgroups that run their units of work two ahead, as the bf16-activation kernel
// does: ragged metadata in LDS, a unit's gather indices fetched two units ahead and its epilogue operands one unit ahead,
// its first K-stage issued before the previous unit's epilogue, tiles claimed from per-XCD queues when they do not
// divide evenly, and an epilogue without branches around stores.  Needs what that scheme needs from the host: at most
// kMetaSlices slices, activations (and their scales) addressable with 32-bit byte offsets, aligned output rows in a
// buffer of less than 2 GiB, no betas / out_alpha / acc_in.
template <int BLKM, int MFW, int NFW, bool SWIGLU, bool MXOUT>
__global__ __launch_bounds__(256) void moe_gemm_mx8p_kernel(const GemmParams p) {
  typedef Frag<32> FR;
  constexpr int FM = 32, NT = 256, BM = MFW * 32, BN = 128 * NFW, KC = 128, NS = 2;
  constexpr int XPITCH = KC + 16;
  constexpr int XBYTES = BM * XPITCH;
  constexpr int XCH = BM / 32;
  // Register rings: weights WD stages deep (stage c uses slot c % WD, loads run WD - 1 stages ahead), activations XD
  // stages deep on their way to LDS.  The stage body is unrolled UNR = lcm(WD, XD, 2) times so that every index is static.
  constexpr int WD = 4, XD = 2, UNR = 4;  // (6 / 3 / 6 fits the registers too and measured 2 % faster on the first GEMM, 3 % slower on the second)
  static_assert(UNR % WD == 0 && UNR % XD == 0 && UNR % 2 == 0, "ring depths divide the unroll factor");
  static_assert(BM <= NT && BN <= NT, "one thread per tile row and per tile column fetches the epilogue operands");
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ int32_t soffs_s[kMetaSlices], ssize_s[kMetaSlices], boffs_s[kMetaSlices + 1];
  __shared__ __attribute__((aligned(16))) float bias_s[2][BN];
  __shared__ float gam_s[2][BM];
  __shared__ int32_t dst_s[2][BM], gidx_s[2][BM];
  __shared__ int next_tile_s[2];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int nw = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 31, h = lane >> 5;
  const int K = p.K, N = p.N;
  const int nst = p.w_nst;
  const int nfr = (N + 31) >> 5;
  const int xc = tid & 7;
  const int xlds0 = (tid >> 3) * XPITCH + xc * 16;  // activation piece j at xlds0 + j*32*XPITCH
  const int kblocks = (K + 31) >> 5;
  const int grid = (int)gridDim.x;
  const bool ragged = p.slice_sizes != nullptr;
  const int nblk = ragged ? p.block_offs[p.n_slices] : 0;
  const int live = ragged ? nblk * p.grid_n : p.total_tiles;
  if (ragged) {
    for (int i = tid; i < p.n_slices; i += NT) {
      soffs_s[i] = p.slice_offs[i];
      ssize_s[i] = p.slice_sizes[i];
      boffs_s[i] = p.block_offs[i];
    }
    if (tid == 0) boffs_s[p.n_slices] = nblk;
  }
  const __amdgpu_buffer_rsrc_t yrsrc = __builtin_amdgcn_make_buffer_rsrc(p.y, 0, p.y_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t ysrsrc = __builtin_amdgcn_make_buffer_rsrc(p.y_mx_scale, 0, MXOUT ? 0x7FFFFFFF : 0, 0x00020000);

  struct Unit {
    int expert, blk_off, blk_rows, pid_n, start_m, pass_off;
    bool valid;
  };
  auto tile_unit = [&](int pid) __attribute__((always_inline)) -> Unit {
    Unit u;
    int eM;
    if (ragged) {
      // tiles are ordered (expert, column tile, row block); the expert is the last slice whose first block is not past
      // block pid / grid_n: a binary search in the block offsets kept in LDS
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
    return u;
  };
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

  // (tiles are dealt statically here: claimed tiles start at different times and drift apart in K, and the workgroups of
  // an XCD then no longer meet each other's activation rows in its L2; measured 3 % slower at the gpt-oss shape)
  constexpr bool dyn = false;
  TileClaimer claimer;
  int round0 = 0;
  int pid, pid_next;
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
  int n_tile = 0;
  if (ragged) __syncthreads();

  // per-unit operand addresses: uniform 64-bit bases plus 32-bit byte offsets per lane
  uint32_t xoff[XCH];   // this thread's row of piece j in x (one byte per element)
  uint32_t xsoff = 0;   // row `tid` in the activation scales
  const uint8_t* wbase[NFW];
  const uint8_t* sbase[NFW];
  const uint32_t lane16 = lane * 16, lr4 = lr * 4;
  auto unit_gather_index = [&](const Unit& u) __attribute__((always_inline)) -> int {
    int row = u.blk_off + u.pass_off + tid;
    row = row < u.blk_off + u.blk_rows ? row : u.blk_off + u.blk_rows - 1;
    const int srow = u.start_m + row;
    return p.gather ? p.gather[srow] : srow;
  };
  auto unit_pointers = [&](const Unit& u, int set) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < XCH; ++j) xoff[j] = (uint32_t)gidx_s[set][(tid >> 3) + 32 * j] * (uint32_t)p.x_stride_m;
    xsoff = (uint32_t)gidx_s[set][tid < BM ? tid : BM - 1] * (uint32_t)p.xs_stride_m;
#pragma unroll
    for (int f = 0; f < NFW; ++f) {
      int F = u.pid_n * (BN / 32) + nw * NFW + f;
      F = F < nfr ? F : nfr - 1;
      wbase[f] = p.w + (int64_t)u.expert * p.w_stride_e + (int64_t)F * nst * 2048;
      sbase[f] = p.w_scale + (int64_t)u.expert * p.ws_stride_e + (int64_t)F * nst * 128;
    }
  };
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
    const int srow = u.start_m + row;
    if (p.gammas) gam_raw = p.gammas_is_f32 ? static_cast<const uint32_t*>(p.gammas)[srow] : (uint32_t)static_cast<const uint16_t*>(p.gammas)[srow];
    if (p.scatter) dst_raw = p.scatter[srow < p.scatter_len ? srow : p.scatter_len - 1];
  };
  auto stage_operands = [&](const Unit& u, int set) __attribute__((always_inline)) {
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
  u32x4_t xreg[XD][XCH];
  // the activation scales of this thread's row for FOUR stages (16 blocks of 32) at a time: the group in use and the one
  // after it, and by how many bytes each load was moved back to stay inside the row (the last group of a row)
  u32x4_t xsq_cur = {}, xsq_nxt = {};
  int gsh_cur = 0, gsh_nxt = 0;
  u32x4_t wraw[WD][NFW][NS];
  uint32_t sd[WD][NFW];
  i32x8_t xf[2][MFW];
  uint32_t xs[2][MFW];

  auto load_x_piece = [&](int j, int s, int slot) __attribute__((always_inline)) {
    int k0 = s * KC + xc * 16;
    k0 = k0 < K - 16 ? k0 : K - 16;
    xreg[slot][j] = *reinterpret_cast<const u32x4_t*>(p.x + (xoff[j] + (uint32_t)k0));
  };
  // One 16-byte load per row and four stages instead of a 4-byte load per row and stage: every lane of such a load owns
  // another row, i.e. another cache line, so the scales, 4 bytes per row and stage, cost as many line look-ups per
  // stage as the 128 bytes of activations per row that they belong to.  (kblocks >= 16: the host's condition.)
  auto load_x_scale_group = [&](int g, u32x4_t& dst, int& gsh) __attribute__((always_inline)) {
    int b0 = g * 16;
    b0 = b0 < kblocks - 16 ? b0 : kblocks - 16;
    __builtin_memcpy(&dst, p.x_mx_scale + (xsoff + (uint32_t)b0), 16);
    gsh = g * 16 - b0;
  };
  auto store_x_piece = [&](int j, int buf, int slot) __attribute__((always_inline)) {
    *reinterpret_cast<u32x4_t*>(lds + buf * XBYTES + xlds0 + j * 32 * XPITCH) = xreg[slot][j];
  };
  // stage d (0..3) of the group held in q: its four scale bytes start 4 d + gsh bytes into q; bytes past q are 2^0
  auto store_x_scale = [&](int buf, const u32x4_t& q, int gsh, int d) __attribute__((always_inline)) {
    const int o = 4 * d + gsh;
    const int idx = o >> 2, sh = (o & 3) * 8;
    auto word = [&](int i) __attribute__((always_inline)) -> uint32_t {
      return i == 0 ? q.x : i == 1 ? q.y : i == 2 ? q.z : i == 3 ? q.w : 0x7F7F7F7Fu;
    };
    const uint64_t wide = ((uint64_t)word(idx + 1) << 32) | word(idx);
    const uint32_t v = (uint32_t)(wide >> sh);
    // (no branch inside the K loop: threads past the tile's rows write into the unused pad bytes of a row)
    const int at = tid < BM ? tid * XPITCH + KC : (tid - BM) * XPITCH + KC + 4;
    *reinterpret_cast<uint32_t*>(lds + buf * XBYTES + at) = v;
  };
  auto load_w = [&](auto slot_c, int s) __attribute__((always_inline)) {
    constexpr int SL = decltype(slot_c)::value;
    s = s < nst ? s : nst - 1;
#pragma unroll
    for (int f = 0; f < NFW; ++f) {
      wraw[SL][f][0] = *reinterpret_cast<const u32x4_t*>(wbase[f] + (int64_t)s * 2048 + lane16);
      wraw[SL][f][1] = *reinterpret_cast<const u32x4_t*>(wbase[f] + (int64_t)s * 2048 + 1024 + lane16);
      sd[SL][f] = *reinterpret_cast<const uint32_t*>(sbase[f] + (int64_t)s * 128 + lr4);
    }
  };
  auto read_xf = [&](int buf, int q, int j, i32x8_t (&out)[MFW]) __attribute__((always_inline)) {
    const uint8_t* a = lds + buf * XBYTES + (j * FM + lr) * XPITCH + q * 32 + h * 16;
    const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(a);
    const u32x4_t hi = *reinterpret_cast<const u32x4_t*>(a + 64);
    out[j] = __builtin_bit_cast(i32x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  auto read_xs = [&](int buf, int j, uint32_t (&out)[MFW]) __attribute__((always_inline)) {
    out[j] = *reinterpret_cast<const uint32_t*>(lds + buf * XBYTES + (j * FM + lr) * XPITCH + KC) >> (16 * h);
  };

  template_int<0> S0;

  auto stage = [&](auto nj_c, auto ws_c, int c) __attribute__((always_inline)) {
    constexpr int NJ = decltype(nj_c)::value;
    constexpr int WSU = decltype(ws_c)::value;  // c % UNR
    constexpr int WS4 = WSU % WD;               // weight ring slot of this stage
    constexpr int PAR = WSU & 1;                // LDS buffer and activation scale set
    using WSL = template_int<(WSU + WD - 1) % WD>;
    constexpr int XS = (WSU + 1) % XD;
    constexpr int NM = NJ * NFW;
    constexpr int NOPS = 2 * NJ + 2;
    uint32_t sdh[NFW];
#pragma unroll
    for (int f = 0; f < NFW; ++f) sdh[f] = sd[WS4][f] >> (16 * h);
    static_for<0, NS>([&](auto q_c) __attribute__((always_inline)) {
      constexpr int q = decltype(q_c)::value;
      constexpr int cur = q & 1, nxt = cur ^ 1;
      auto op = [&](auto o_c) __attribute__((always_inline)) {
        constexpr int o = decltype(o_c)::value;
        if constexpr (o < NJ) {
          if constexpr (q == 0) {
            read_xf(PAR, 1, o, xf[nxt]);
          } else {
            read_xf(PAR ^ 1, 0, o, xf[nxt]);
            read_xs(PAR ^ 1, o, xs[PAR ^ 1]);
          }
        } else if constexpr (o < 2 * NJ) {
          if constexpr (q == 0) {
            constexpr int j = o - NJ;
            store_x_piece(j, PAR ^ 1, XS);
            load_x_piece(j, c + 1 + XD, XS);
          }
        } else if constexpr (o == 2 * NJ) {
          if constexpr (q == 0) {
            // stage c + 1's scales go to LDS; c is a multiple of UNR = 4 at unroll position 0, so stage c + 1 is stage
            // (WSU + 1) % 4 of its group.  Position 0 takes over the group requested at position 1 of the round before,
            // position 3 already serves the next round's first stage from it.
            constexpr int D = (WSU + 1) & 3;
            if constexpr (WSU == 0) {
              xsq_cur = xsq_nxt;
              gsh_cur = gsh_nxt;
            }
            if constexpr (D == 0)
              store_x_scale(PAR ^ 1, xsq_nxt, gsh_nxt, 0);
            else
              store_x_scale(PAR ^ 1, xsq_cur, gsh_cur, D);
            if constexpr (WSU == 1) load_x_scale_group((c + 3) >> 2, xsq_nxt, gsh_nxt);
          }
        } else {
          if constexpr (q == 0) load_w(WSL{}, c + WD - 1);
        }
      };
      static_for<0, NM>([&](auto m_c) __attribute__((always_inline)) {
        constexpr int m = decltype(m_c)::value;
        constexpr int j = m / NFW, f = m % NFW;
        const u32x4_t wv = wraw[WS4][f][q];
        // (an fp4 operand is the low four of the eight registers the builtin's type has; the others stay undefined)
        const i32x8_t a = __builtin_bit_cast(i32x8_t, __builtin_shufflevector(wv, wv, 0, 1, 2, 3, -1, -1, -1, -1));
        acc[f][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, xf[cur][j], acc[f][j], 4 /* A: e2m1 */, 0 /* B: e4m3 */, q, (int)sdh[f], q,
                                                                     (int)xs[PAR][j]);
        if constexpr (q == NS - 1 && m == 0) {
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        }
        static_for<(m * NOPS) / NM, ((m + 1) * NOPS) / NM>(op);
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };

  // stage 0 of a unit (every piece, so that the number of loads does not depend on the unit): issued before the
  // previous unit's epilogue arithmetic
  auto first_loads = [&]() __attribute__((always_inline)) {
    static_for<0, XCH>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 0, 0); });
    load_x_scale_group(0, xsq_nxt, gsh_nxt);
    __builtin_amdgcn_sched_barrier(0);
    load_w(S0, 0);
    __builtin_amdgcn_sched_barrier(0);
  };

  int up = 0;
  Unit cur_unit;
  int resolve_slot = -1;
  auto run = [&](auto nj_c) __attribute__((always_inline)) {
    constexpr int NJ = decltype(nj_c)::value;
    [[maybe_unused]] const long long t_run = MX8_T();
    // the loads left in flight at the loop header are in the order the steady state leaves them in at the top of a
    // stage: activations, their scales, weights of stage 1, then of stage 2
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) { store_x_piece(decltype(jc)::value, 0, 0); });
    store_x_scale(0, xsq_nxt, gsh_nxt, 0);
    xsq_cur = xsq_nxt;
    gsh_cur = gsh_nxt;
    __builtin_amdgcn_sched_barrier(0);
    // what the stages -max(XD, WD - 2) .. -1 would have issued had the loop been running: stage i requests the activations
    // of stage i + 1 + XD, then the weights of stage i + WD - 1 (this unit's: indices from 1 on)
    constexpr int LEAD = XD > WD - 2 ? XD : WD - 2;
    static_for<0, LEAD>([&](auto i_c) __attribute__((always_inline)) {
      constexpr int i = decltype(i_c)::value - LEAD;
      constexpr int sx = i + 1 + XD, sw = i + WD - 1;
      if constexpr (sx >= 1) {
        static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, sx, sx % XD); });
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (sw >= 1) {
        load_w(template_int<sw % WD>{}, sw);
        __builtin_amdgcn_sched_barrier(0);
      }
    });
    stage_operands(cur_unit, up);
    if (resolve_slot >= 0 && tid == 0) next_tile_s[resolve_slot] = claimer.resolve();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) {
      read_xf(0, 0, decltype(jc)::value, xf[0]);
      read_xs(0, decltype(jc)::value, xs[0]);
    });
    __builtin_amdgcn_sched_barrier(0);
    [[maybe_unused]] const long long t_loop = MX8_T();
    MX8_ADD(0, t_loop - t_run);
    int c = 0;
    for (; c + UNR - 1 < nst; c += UNR)
      static_for<0, UNR>([&](auto u_c) __attribute__((always_inline)) { stage(nj_c, u_c, c + decltype(u_c)::value); });
    static_for<0, UNR - 1>([&](auto u_c) __attribute__((always_inline)) {
      if (c + decltype(u_c)::value < nst) stage(nj_c, u_c, c + decltype(u_c)::value);
    });
    MX8_ADD(1, MX8_T() - t_loop);
    MX8_ADD(5, nst);
  };

  [[maybe_unused]] const long long t_kernel = MX8_T();
  if (pid >= 0) {
    Unit& cur = cur_unit;
    cur = tile_unit(pid);
    Unit nxt = advance(cur, pid_next);
    if (tid < BM) gidx_s[1][tid] = unit_gather_index(cur);
    __syncthreads();
    unit_pointers(cur, 1);
    unit_operands(cur);
    if (nxt.valid && tid < BM) gidx_v = unit_gather_index(nxt);
    if (dyn && pid_next >= 0) {
      claimer.issue();
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
      const int nj = (rows + FM - 1) / FM;
      static_for<1, MFW + 1>([&](auto n_c) __attribute__((always_inline)) {
        if (nj == decltype(n_c)::value) run(n_c);
      });
      resolve_slot = -1;
      [[maybe_unused]] const long long t_prep = MX8_T();

      const int wcol = nw * NFW * FM;
      const int ncol0 = cur.pid_n * BN + wcol;
      Unit nxt2 = nxt;
      if (nxt.valid) {
        if (cur.pass_off + BM >= cur.blk_rows) {
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
        unit_operands(nxt);
        if (nxt2.valid && tid < BM) gidx_v = unit_gather_index(nxt2);
        __builtin_amdgcn_sched_barrier(0);
        unit_pointers(nxt, up);
        first_loads();
      }
      [[maybe_unused]] const long long t_epi = MX8_T();
      MX8_ADD(2, t_epi - t_prep);
      if constexpr (MXOUT)
        staged_mx_epilogue<MFW, NFW, SWIGLU>(p, acc, yrsrc, ysrsrc, bias_s[up], gam_s[up], dst_s[up], wcol, ncol0, lr, h);
      else
        staged_epilogue<1, MFW, NFW, NFW, SWIGLU, true>(p, acc, yrsrc, bias_s[up], gam_s[up], dst_s[up], wcol, ncol0, 0, lr, h);
      MX8_ADD(3, MX8_T() - t_epi);
      MX8_ADD(4, 1);
      if (!nxt.valid) break;
      cur = nxt;
      nxt = nxt2;
      up ^= 1;
    }
  }
  if (dyn) claimer.finish();
  MX8_ADD(6, MX8_T() - t_kernel);
}

template <int BLKM, int MFW, int NFW>
int32_t launch_mx8n(const GemmParams& p, int grid_m, bool swiglu, bool mxout, hipStream_t st) {
  constexpr int LDS_BYTES = 2 * MFW * 32 * (128 + 16);
  GemmParams q = p;
  q.grid_n = (int)cdiv(p.N, 128 * NFW);
  int64_t grid = (int64_t)grid_m * q.grid_n;
  if (grid <= 0) return TK_OK;
  if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: grid too large");
  q.total_tiles = (int32_t)grid;
  const int64_t resident = (int64_t)busy_cu_count(p.idle_cus);  // persistent grid, one workgroup per CU
  if (grid > resident) grid = resident;
  auto launch = [&](auto kern) -> int32_t {
    if (const int32_t rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), LDS_BYTES)) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), LDS_BYTES, st, q);
    return check_launch("moe_gemm_mx8n_kernel");
  };
  if (p.y_bytes != 0) {
    // (the host found what the persistent form needs)
    if (swiglu && mxout) return launch(moe_gemm_mx8p_kernel<BLKM, MFW, NFW, true, true>);
    if (swiglu) return launch(moe_gemm_mx8p_kernel<BLKM, MFW, NFW, true, false>);
    if (mxout) return launch(moe_gemm_mx8p_kernel<BLKM, MFW, NFW, false, true>);
    return launch(moe_gemm_mx8p_kernel<BLKM, MFW, NFW, false, false>);
  }
  if (swiglu && mxout) return launch(moe_gemm_mx8n_kernel<BLKM, MFW, NFW, true, true>);
  if (swiglu) return launch(moe_gemm_mx8n_kernel<BLKM, MFW, NFW, true, false>);
  if (mxout) return launch(moe_gemm_mx8n_kernel<BLKM, MFW, NFW, false, true>);
  return launch(moe_gemm_mx8n_kernel<BLKM, MFW, NFW, false, false>);
}

}  // namespace

#ifdef TK_MX8_STAMPS
extern "C" int32_t tk_debug_mx8_stamps(long long* host_out, int32_t clear) {
  if (clear) {
    static long long zeros[1024 * 8];
    return hipMemcpyToSymbol(HIP_SYMBOL(mx8_stamps), zeros, sizeof(zeros)) == hipSuccess ? 0 : 3;
  }
  return hipMemcpyFromSymbol(host_out, HIP_SYMBOL(mx8_stamps), sizeof(long long) * 1024 * 8) == hipSuccess ? 0 : 3;
}
#endif

int32_t gemm_launch_mx8n(const GemmParams& p, int block_m, int grid_m, bool swiglu, bool mx_out, hipStream_t st) {
  //                                       BLKM MFW NFW
  if (block_m == 256) return launch_mx8n<256, 5, 2>(p, grid_m, swiglu, mx_out, st);
  return launch_mx8n<128, 4, 2>(p, grid_m, swiglu, mx_out, st);
}

}  // namespace tk
