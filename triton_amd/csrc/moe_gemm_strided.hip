// Ragged (grouped) expert GEMM for gfx950 with fused gather, MX dequantisation, bias, swiglu, gate
// scaling and scatter.
//
//   Y[dst(r), :] = act( (X[src(r), :] @ W[e(r)]) * sx[src(r)] * sw[e(r), :] + bias[e(r), :] ) * gamma[r]
//
// Mapping onto CDNA4:
//   * one workgroup (WM x WN wave64s) computes BM = WM*MFW*FM rows of ONE expert by BN = WN*NFW*FM
//     output columns (FM = 16 or 32, the MFMA fragment edge); the K loop runs in stages of KC = 128*KS;
//   * the MFMA is issued "transposed": the A operand is a 16(n) x 32(k) fragment of W^T and the B
//     operand a 32(k) x 16(m) fragment of X^T, so a lane's 4 accumulator registers are 4 CONSECUTIVE
//     output columns of one row (swiglu's (gate, linear) column pairs are lane-local) and both
//     operands want K-contiguous data, which is how activations ([rows, K]) and the reference's MX
//     weights ([E, N, K/2] in memory) are stored;
//   * both operands are staged through LDS, double buffered, with global loads issued one stage ahead
//     into registers.  Loads are shaped for the texture-address unit: 16 consecutive lanes fetch 256
//     contiguous bytes of one activation row, 4 consecutive lanes the 64 bytes one weight column
//     contributes to a stage; LDS rows are padded by 16 B so the ds_read_b128 of 16 rows / columns is
//     bank-conflict free.  MXFP4 stays packed in LDS (4 bits per weight) together with its e8m0 scales
//     and is expanded in registers by v_cvt_scalef32_pk_bf16_fp4 right before the MFMA;
//   * the rows of a tile are dealt to the WM row-waves in interleaved 16-row fragments and fragments
//     past the expert's last row are skipped, so a nearly empty row block costs almost no MFMA time.
#include "gemm_common.h"

namespace tk {
namespace {

template <int WK, int FM, int WM, int WN, int MFW, int NFW, int KS, bool SWIGLU>
__global__ __launch_bounds__(WM * WN * 64) void moe_gemm_kernel(const GemmParams p) {
  typedef Frag<FM> FR;
  constexpr int NT = WM * WN * 64;
  constexpr int BM = WM * MFW * FM;
  constexpr int BN = WN * NFW * FM;
  constexpr int KC = 128 * KS;  // K elements per pipeline stage
  constexpr int NG = 64 / FM;   // k-groups of lanes
  constexpr int KG = 128 / NG;  // k per group per 128-wide sub-stage
  constexpr int SPS = KG / 8;   // MFMA steps per sub-stage
  constexpr bool MX = WK == WK_MXFP4;
  constexpr bool F8 = WK == WK_FP8;  // e4m3 weights AND e4m3 activations, both expanded to bf16 for the MFMA
  constexpr int XE = F8 ? 16 : 8;    // activation elements per 16-byte global piece
  constexpr int XPITCH = KC * 2 + 16;                    // bytes per activation row in LDS
  constexpr int WROW = MX ? KC / 2 : (F8 ? KC : KC * 2);  // weight bytes per column per stage
  constexpr int WPITCH = WROW + 16;                      // MX: the pad holds the KC/32 scale bytes
  constexpr int XBYTES = BM * XPITCH;
  constexpr int STAGE = XBYTES + BN * WPITCH;
  constexpr int XPIECES = BM * (KC / XE);                // 16-byte global pieces per stage
  constexpr int WPIECES = BN * (WROW / 16);
  constexpr int XCH = (XPIECES + NT - 1) / NT;
  constexpr int WCH = (WPIECES + NT - 1) / NT;
  constexpr int SCH = MX ? (BN * KS + NT - 1) / NT : 1;  // scale dwords (4 blocks = 128 k each)
  constexpr bool XFULL = XPIECES % NT == 0, WFULL = WPIECES % NT == 0, SFULL = (BN * KS) % NT == 0;
  static_assert(2 * STAGE <= 160 * 1024, "LDS budget");

  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  int expert, off_m, start_m, eM, pid_n;
  if (p.slice_sizes) {
    // The grid is an upper bound; renumber only the live tiles so that every XCD gets an equal share.
    const int live = p.block_offs[p.n_slices] * p.grid_n;
    if ((int)blockIdx.x >= live) return;
    const int pid = xcd_remap(blockIdx.x, live);
    // Tiles are ordered (expert, column tile, row block): the row blocks of one expert that share a column
    // tile get consecutive ids, run at the same time on one XCD and stream the same weights through its L2.
    expert = p.block_sched[pid / p.grid_n] & 0xFFFF;
    const int first = p.block_offs[expert];
    const int nb = p.block_offs[expert + 1] - first;
    const int local = pid - first * p.grid_n;
    pid_n = local / nb;
    off_m = (local - pid_n * nb) * BM;
    start_m = p.slice_offs[expert];
    eM = p.slice_sizes[expert];
  } else {
    const int pid = xcd_remap(blockIdx.x, gridDim.x);
    pid_n = pid % p.grid_n;
    expert = 0;
    off_m = (pid / p.grid_n) * BM;
    start_m = 0;
    eM = p.M;
  }
  const int rows = (eM - off_m) < BM ? (eM - off_m) : BM;  // valid rows of this tile (>= 1)
  const int nfrag_m = (rows + FM - 1) / FM;                // row fragments that hold valid rows
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int mw = wave % WM, nw = wave / WM;
  const int lr = lane % FM, h = lane / FM;
  const int K = p.K, N = p.N;
  // fragment j of this wave covers tile rows (j*WM + mw)*FM .. +FM; fragments past the last valid row are skipped
  int jcount = 0;
#pragma unroll
  for (int j = 0; j < MFW; ++j) jcount += ((j * WM + mw) < nfrag_m) ? 1 : 0;

  // ---- global -> register staging: this thread's 16-byte pieces -----------------------------
  const uint8_t* xptr[XCH];
  int xk[XCH], xlds[XCH];
  bool xok[XCH];
#pragma unroll
  for (int j = 0; j < XCH; ++j) {
    const int id = tid + NT * j;
    const int r = (id / (KC / XE)) % BM, c = id % (KC / XE);
    xok[j] = (XFULL || id < XPIECES) && r < nfrag_m * FM;  // fragments without valid rows are never read
    int row = off_m + r;
    row = row < eM ? row : eM - 1;
    const int64_t src = p.gather ? (int64_t)p.gather[start_m + row] : (int64_t)(start_m + row);
    xptr[j] = p.x + (src * p.x_stride_m + c * XE) * (F8 ? 1 : 2);
    xk[j] = c * XE;
    xlds[j] = r * XPITCH + c * XE * 2;
  }
  const uint8_t* wptr[WCH];
  int wk[WCH], wlds[WCH];
  bool wok[WCH];
  const int n_tile = pid_n * BN;
#pragma unroll
  for (int j = 0; j < WCH; ++j) {
    const int id = tid + NT * j;
    wok[j] = WFULL || id < WPIECES;
    const int col = (id / (WROW / 16)) % BN, part = id % (WROW / 16);
    int n = n_tile + col;
    n = n < N ? n : N - 1;  // columns past N are computed from a valid column and dropped in the epilogue
    wptr[j] = p.w + (int64_t)expert * p.w_stride_e + (int64_t)n * p.w_stride_n + part * 16;
    wk[j] = MX ? part * 32 : (F8 ? part * 16 : part * 8);
    wlds[j] = XBYTES + col * WPITCH + part * 16;
  }
  const uint8_t* sptr[SCH];
  int sk[SCH], slds[SCH];
  bool sok[SCH];
  if constexpr (MX) {
#pragma unroll
    for (int j = 0; j < SCH; ++j) {
      const int id = tid + NT * j;
      sok[j] = SFULL || id < BN * KS;
      const int col = (id / KS) % BN, part = id % KS;
      int n = n_tile + col;
      n = n < N ? n : N - 1;
      sptr[j] = p.w_scale + (int64_t)expert * p.ws_stride_e + (int64_t)n * p.ws_stride_n + part * 4;
      sk[j] = part * 128;
      slds[j] = XBYTES + col * WPITCH + WROW + part * 4;
    }
  }

  typename FR::acc_t acc[NFW][MFW];
#pragma unroll
  for (int f = 0; f < NFW; ++f)
#pragma unroll
    for (int j = 0; j < MFW; ++j)
#pragma unroll
      for (int i = 0; i < FR::NACC; ++i) acc[f][j][i] = 0.f;

  uint4 xreg[XCH];
  uint4 wreg[WCH];
  uint32_t sreg[SCH];

  // TAIL = the stage may reach past K: pieces beyond K are zero-filled (zero weights x finite activations)
  auto load_stage = [&](auto tail_c, int kc) __attribute__((always_inline)) {
    constexpr bool TAIL = decltype(tail_c)::value;
#pragma unroll
    for (int j = 0; j < XCH; ++j) {
      if (xok[j] && (!TAIL || kc + xk[j] < K))
        xreg[j] = *reinterpret_cast<const uint4*>(xptr[j] + kc * (F8 ? 1 : 2));
      else
        xreg[j] = make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < WCH; ++j) {
      if ((WFULL || wok[j]) && (!TAIL || kc + wk[j] < K))
        wreg[j] = *reinterpret_cast<const uint4*>(wptr[j] + (MX ? kc / 2 : (F8 ? kc : kc * 2)));
      else
        wreg[j] = make_uint4(0, 0, 0, 0);
    }
    if constexpr (MX) {
#pragma unroll
      for (int j = 0; j < SCH; ++j) {
        if (!(SFULL || sok[j])) {
          sreg[j] = 0x7F7F7F7Fu;
        } else if (!TAIL) {
          uint32_t v;
          __builtin_memcpy(&v, sptr[j] + kc / 32, 4);  // 4 consecutive e8m0 bytes, any alignment
          sreg[j] = v;
        } else {
          uint32_t v = 0;
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            const int k0 = kc + sk[j] + 32 * b;
            const uint32_t byte = k0 < K ? (uint32_t)sptr[j][kc / 32 + b] : 127u;
            v |= byte << (8 * b);
          }
          sreg[j] = v;
        }
      }
    }
  };
  auto store_stage = [&](int buf) __attribute__((always_inline)) {
    uint8_t* base = lds + buf * STAGE;
#pragma unroll
    for (int j = 0; j < XCH; ++j)
      if (xok[j]) {
        if constexpr (F8) {  // 16 e4m3 -> 16 bf16 (exact)
          const uint32_t w4[4] = {xreg[j].x, xreg[j].y, xreg[j].z, xreg[j].w};
          uint32_t o[8];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            o[2 * q] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w4[q], 1.0f, false));
            o[2 * q + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w4[q], 1.0f, true));
          }
          *reinterpret_cast<uint4*>(base + xlds[j]) = make_uint4(o[0], o[1], o[2], o[3]);
          *reinterpret_cast<uint4*>(base + xlds[j] + 16) = make_uint4(o[4], o[5], o[6], o[7]);
        } else {
          *reinterpret_cast<uint4*>(base + xlds[j]) = xreg[j];
        }
      }
#pragma unroll
    for (int j = 0; j < WCH; ++j)
      if (WFULL || wok[j]) *reinterpret_cast<uint4*>(base + wlds[j]) = wreg[j];
    if constexpr (MX) {
#pragma unroll
      for (int j = 0; j < SCH; ++j)
        if (SFULL || sok[j]) *reinterpret_cast<uint32_t*>(base + slds[j]) = sreg[j];
    }
  };
  // MFMA step t of a stage: sub-stage s = t / SPS, i = t % SPS; lane group h supplies k = s*128 + h*KG + i*8 .. +8
  auto read_xf = [&](const uint8_t* base, int t, bf16x8_t (&xf)[MFW]) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < MFW; ++j)
      xf[j] = *reinterpret_cast<const bf16x8_t*>(base + ((j * WM + mw) * FM + lr) * XPITCH +
                                                  ((t / SPS) * 128 + h * KG + (t % SPS) * 8) * 2);
  };
  // FULL: every row fragment of this wave holds valid rows; the body is then one straight-line block in
  // which the scheduler is told to alternate MFMAs with the dequantisation / LDS reads of the next step.
  auto compute = [&](auto full_c, int buf) __attribute__((always_inline)) {
    constexpr bool FULL = decltype(full_c)::value;
    const uint8_t* base = lds + buf * STAGE;
    const uint8_t* wbase = base + XBYTES + (nw * NFW * FM + lr) * WPITCH;
    constexpr int STEPS = KS * SPS;
    bf16x8_t xf[2][MFW];
    bf16x8_t wf[2][NFW];
    uint32_t wraw[NFW][KG / 8];  // KG e2m1 values of this lane's column (current sub-stage)
    uint32_t sd[NFW];            // the sub-stage's 4 scale bytes of this lane's column
    auto read_w = [&](int sub) __attribute__((always_inline)) {
      if constexpr (MX) {
#pragma unroll
        for (int f = 0; f < NFW; ++f) {
#pragma unroll
          for (int q = 0; q < KG / 32; ++q) {
            const uint4 v = *reinterpret_cast<const uint4*>(wbase + f * FM * WPITCH + sub * 64 + h * (KG / 2) + q * 16);
            wraw[f][4 * q + 0] = v.x;
            wraw[f][4 * q + 1] = v.y;
            wraw[f][4 * q + 2] = v.z;
            wraw[f][4 * q + 3] = v.w;
          }
          sd[f] = *reinterpret_cast<const uint32_t*>(wbase + f * FM * WPITCH + WROW + sub * 4);
        }
      }
    };
    auto make_wf = [&](int t, bf16x8_t (&out)[NFW]) __attribute__((always_inline)) {
      const int sub = t / SPS, i = t % SPS;
#pragma unroll
      for (int f = 0; f < NFW; ++f) {
        if constexpr (MX) {
          const int blk = h * (KG / 32) + i / 4;  // MX block (of the sub-stage's 4) this step's 8 values lie in
          out[f] = dequant8(wraw[f][i], bits_f32(((sd[f] >> (8 * blk)) & 0xFFu) << 23));
        } else {
          if constexpr (F8) {  // 8 e4m3 -> 8 bf16 (exact)
            const uint2 raw = *reinterpret_cast<const uint2*>(wbase + f * FM * WPITCH + sub * 128 + h * KG + i * 8);
            const bf16x2_t a = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.x, 1.0f, false);
            const bf16x2_t b = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.x, 1.0f, true);
            const bf16x2_t c2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.y, 1.0f, false);
            const bf16x2_t d2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.y, 1.0f, true);
            out[f] = bf16x8_t{a[0], a[1], b[0], b[1], c2[0], c2[1], d2[0], d2[1]};
          } else {
            out[f] = *reinterpret_cast<const bf16x8_t*>(wbase + f * FM * WPITCH + (sub * 128 + h * KG + i * 8) * 2);
          }
        }
      }
    };
    read_w(0);
    read_xf(base, 0, xf[0]);
    make_wf(0, wf[0]);
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
      const int cur = t & 1, nxt = cur ^ 1;
      if (t + 1 < STEPS) {
        if ((t + 1) % SPS == 0) read_w((t + 1) / SPS);
        read_xf(base, t + 1, xf[nxt]);
        make_wf(t + 1, wf[nxt]);
      }
#pragma unroll
      for (int j = 0; j < MFW; ++j) {
        if (FULL || j < jcount) {
#pragma unroll
          for (int f = 0; f < NFW; ++f) {
            if constexpr (WK == WK_F16)
              acc[f][j] = FR::mma_f16(wf[cur][f], xf[cur][j], acc[f][j]);
            else
              acc[f][j] = FR::mma(wf[cur][f], xf[cur][j], acc[f][j]);
          }
        }
      }
      if constexpr (FULL) {
        // per MFMA: the share of the next step's VALU work (4 conversions per weight fragment) and LDS reads
        constexpr int NM = MFW * NFW;
        constexpr int VPM = MX ? (4 * NFW + NM - 1) / NM + 1 : 0;
#pragma unroll
        for (int m = 0; m < NM; ++m) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (m < MFW + (MX ? 0 : NFW)) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          if (VPM) __builtin_amdgcn_sched_group_barrier(0x002, VPM, 0);
        }
      }
    }
  };
  using T_ = std::true_type;
  using F_ = std::false_type;
  auto compute_any = [&](int buf) __attribute__((always_inline)) {
    if (jcount == MFW)
      compute(T_{}, buf);
    else
      compute(F_{}, buf);
  };

  // Pipeline: registers hold stage c+1 (loaded while stage c-1 was computed); at the top of stage c they go
  // to the other LDS buffer, the loads of stage c+2 are issued, then stage c is computed from LDS.
  const int nstages = (K + KC - 1) / KC;
  const int nfull = K / KC;  // stages that lie entirely below K
  auto load_any = [&](int cs) __attribute__((always_inline)) {
    if (cs < nfull)
      load_stage(F_{}, cs * KC);
    else
      load_stage(T_{}, cs * KC);
  };
  load_any(0);
  store_stage(0);
  if (nstages > 1) load_any(1);
  __syncthreads();
  for (int c = 0; c < nstages; ++c) {
    if (c + 1 < nstages) store_stage((c + 1) & 1);
    if (c + 2 < nstages) load_any(c + 2);
    compute_any(c & 1);
    __syncthreads();
  }

  gemm_epilogue<FM, WM, MFW, NFW, SWIGLU, WK == WK_F16>(p, acc, expert, off_m, start_m, eM, n_tile + nw * NFW * FM, n_tile + BN <= N, mw, lr, h);
}
template <int WK, int FM, int WM, int WN, int MFW, int NFW, int KS>
int32_t launch_cfg(const GemmParams& p, int grid_m, bool swiglu, hipStream_t st) {
  constexpr int BM = WM * MFW * FM;
  constexpr int BN = WN * NFW * FM;
  constexpr int KC = 128 * KS;
  constexpr int WROW = WK == WK_MXFP4 ? KC / 2 : (WK == WK_FP8 ? KC : KC * 2);
  constexpr int LDS_BYTES = 2 * (BM * (KC * 2 + 16) + BN * (WROW + 16));
  GemmParams q = p;
  q.grid_n = (int)cdiv(p.N, BN);
  const int64_t grid = (int64_t)grid_m * q.grid_n;
  if (grid <= 0) return TK_OK;
  if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: grid too large");
  auto launch = [&](auto kern) -> int32_t {
    if (const int32_t rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), LDS_BYTES)) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(WM * WN * 64), LDS_BYTES, st, q);
    return check_launch("moe_gemm_kernel");
  };
  if (swiglu) return launch(moe_gemm_kernel<WK, FM, WM, WN, MFW, NFW, KS, true>);
  return launch(moe_gemm_kernel<WK, FM, WM, WN, MFW, NFW, KS, false>);
}

template <int WK>
int32_t launch_wk(const GemmParams& p, int block_m, int grid_m, bool swiglu, hipStream_t st) {
  //                      FM  WM WN MFW NFW KS
  if constexpr (WK == WK_MXFP4) {
    switch (block_m) {
      case 16:
        return launch_cfg<WK, 16, 1, 4, 1, 2, 2>(p, grid_m, swiglu, st);
      case 32:
        return launch_cfg<WK, 16, 1, 4, 2, 2, 2>(p, grid_m, swiglu, st);
      case 64:
        return launch_cfg<WK, 32, 2, 2, 1, 4, 1>(p, grid_m, swiglu, st);
      case 128:
        return launch_cfg<WK, 32, 2, 2, 2, 4, 1>(p, grid_m, swiglu, st);
    }
  } else if constexpr (WK == WK_FP8) {
    switch (block_m) {
      case 16:
        return launch_cfg<WK, 16, 1, 4, 1, 2, 2>(p, grid_m, swiglu, st);
      case 32:
        return launch_cfg<WK, 16, 1, 4, 2, 2, 2>(p, grid_m, swiglu, st);
      case 64:
        return launch_cfg<WK, 32, 2, 2, 1, 4, 1>(p, grid_m, swiglu, st);
      case 128:
        return launch_cfg<WK, 32, 2, 2, 2, 4, 1>(p, grid_m, swiglu, st);
    }
  } else {
    switch (block_m) {
      case 16:
        return launch_cfg<WK, 16, 1, 4, 1, 2, 1>(p, grid_m, swiglu, st);
      case 32:
        return launch_cfg<WK, 16, 1, 4, 2, 2, 1>(p, grid_m, swiglu, st);
      case 64:
        return launch_cfg<WK, 32, 2, 2, 1, 2, 1>(p, grid_m, swiglu, st);
      case 128:
        return launch_cfg<WK, 32, 2, 2, 2, 2, 1>(p, grid_m, swiglu, st);
    }
  }
  return fail(TK_ERR_INVALID, "tk_moe_gemm: block_m must be 16, 32, 64 or 128 (got %d)", block_m);
}

}  // namespace

int32_t gemm_launch_strided(const GemmParams& p, int wk, int block_m, int grid_m, bool swiglu, hipStream_t st) {
  switch (wk) {
    case WK_MXFP4:
      return launch_wk<WK_MXFP4>(p, block_m, grid_m, swiglu, st);
    case WK_BF16:
      return launch_wk<WK_BF16>(p, block_m, grid_m, swiglu, st);
    case WK_F16:
      return launch_wk<WK_F16>(p, block_m, grid_m, swiglu, st);
    case WK_FP8:
      return launch_wk<WK_FP8>(p, block_m, grid_m, swiglu, st);
  }
  return fail(TK_ERR_INVALID, "tk_moe_gemm: bad weight kind %d", wk);
}

}  // namespace tk
