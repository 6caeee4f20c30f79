// A whole decode-sized MoE FFN layer in ONE launch: router -> gather-GEMM (+bias, swiglu) -> scatter-GEMM (+bias,
// gate weight) -> top-k combine, for a handful of tokens (T * k <= 256 routed rows) over tiled MXFP4 expert weights.
//
// At these sizes the layer is a stream of the active experts' weights (13 MB per expert at the gpt-oss shape) read
// once from HBM; three launches spend a third of their time on launch boundaries and on the serial router in front
// of the first weight byte.  Here the grid is persistent and co-resident (one or two workgroups per CU):
//
//   1. EVERY workgroup routes all T tokens itself (the logits are a few KiB): top-k by wave-wide max rounds, softmax,
//      expert histogram, stable expert-sorted row order - into LDS, no global round trip, no dependence on others.
//   2. The work is cut into units = (active expert, 16-row block, 32-column weight fragment) of GEMM 1 followed by
//      those of GEMM 2; every workgroup takes an equal contiguous share of each list, derived from the LDS tables.
//   3. The NW waves of a workgroup split the K-stages of a unit (K-slices of XS stages); a wave keeps its slice of the
//      block's activation rows in REGISTERS for as long as the (expert, row block) stays the same, so the inner loop
//      is: 2 KiB weight block global -> registers (ring, one unit ahead), e2m1 -> bf16 in registers, 16x16x32 MFMA.
//      The slices meet in LDS once per unit (one barrier); the waves take turns at summing them and running the epilogue.
//   4. GEMM 1 writes its swiglu'd rows (bf16) to a scratch tensor h with write-through stores; a workgroup that has
//      finished its GEMM-1 share counts its units in at a per-expert counter.  GEMM-2 units of an expert wait for that
//      counter (their weight blocks are already on their way) and read h around the L2 (the eight XCDs' L2s are not
//      coherent with each other).
//   5. GEMM 2 writes gate-weighted rows to y [T*k, N]; when a workgroup has finished its share it counts every
//      (token, fragment) it wrote in, and whoever completes a token's k rows sums them in j order in fp32 (what
//      `reduce` does after the reference's scatter, reduce.py:1143-1165) and writes the token's output row.
//   6. The last workgroup to finish clears the counters, so the workspace is ready for the next launch.
//
// Every wait is bounded: a spin that exceeds `spin_limit` polls raises the error word of the workspace and goes on
// (the result is then wrong, but every wave exits).
#include "gemm_common.h"
#include "route_common.h"

namespace tk {
namespace {

constexpr int kDecMaxRows = TK_DECODE_MAX_ROWS;        // T * k
constexpr int kDecMaxExperts = TK_DECODE_MAX_EXPERTS;  // one expert per thread in the placement pass
constexpr int kDecMaxUnits = 192;                      // units of one workgroup (the host bounds it)
constexpr int kDecNW = 8;                              // waves per workgroup = K-slices of a unit
constexpr int kDecXS = 3;                              // K-stages (of 128) per slice: K <= NW * XS * 128 = 3072
constexpr int kDecRing = 3;                            // units of weight blocks a wave holds or has requested
constexpr int kDecBlockStride = 32;                    // words between two row blocks' counters (a cache line each)
constexpr int kDecBlockWords = (kDecMaxRows + kDecMaxRows / 16) * kDecBlockStride;  // 16-row blocks: at most min(E, R) + R / 16

struct DecodeParams {
  const uint8_t* x;  // bf16 [T, K1]
  int64_t x_stride;  // elements
  uint32_t x_bytes;  // extent of x (the rows are read through a buffer resource)
  const void* logits;
  int64_t logits_stride;
  int32_t logits_is_bf16;
  int32_t T, E, k, apply_softmax;
  const uint8_t* w1;
  const uint8_t* w1s;
  int64_t w1_stride_e, w1s_stride_e;  // bytes
  const void* b1;
  int64_t b1_stride_e;
  int32_t b1_is_f32;
  const uint8_t* w2;
  const uint8_t* w2s;
  int64_t w2_stride_e, w2s_stride_e;
  const void* b2;
  int64_t b2_stride_e;
  int32_t b2_is_f32;
  int32_t K1, N1, K2, N2;  // K2 = N1 / 2
  int32_t nst1, nst2, nfr1, nfr2;
  float alpha, limit;
  int32_t has_limit;
  uint16_t* h;      // scratch [T*k, K2] bf16, expert-sorted rows
  uint16_t* y;      // scratch [T*k, N2] bf16, flat rows t*k + j
  int32_t* sync;    // [0] finished workgroups, [1] error word, then kDecBlockWords GEMM-1 units done per row block, then [T*nfr2] arrivals
  uint16_t* out;    // [T, N2] bf16
  int64_t out_stride;
  int16_t* indx_out;  // optional [T, k]
  float* vals_out;    // optional [T, k]
  int32_t spin_limit;
};

struct DecUnit {
  const uint8_t* w;  // first K-stage of the unit's weight fragment
  const uint8_t* s;
  int32_t key;       // phase << 24 | expert slot a << 8 | row block
  int32_t frag;      // column fragment F
};

#ifdef TK_DEC_STAMPS
__device__ long long dec_stamps[1024][20];
#define DEC_STAMP(n) do { if (threadIdx.x == 0) dec_stamps[blockIdx.x][n] = (long long)__builtin_amdgcn_s_memrealtime(); } while (0)
// end of unit i's K loop in every workgroup (rows 512 + 2 * workgroup of the table, 20 columns x 2 rows each)
#define DEC_UNIT_STAMP(i) do { if (threadIdx.x == 0 && blockIdx.x < 256 && (i) < 40) dec_stamps[512 + blockIdx.x * 2 + (i) / 20][(i) % 20] = (long long)__builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define DEC_UNIT_STAMP(i) do {} while (0)
#define DEC_STAMP(n) do {} while (0)
#endif

constexpr int kThrough = 1 | 16;  // aux bits of the buffer instructions: sc0 | sc1 (write through / read around the L2)

// ONCE: no expert has more than one row block (the host knows it from T <= 16: a token's k experts differ), so every
// weight byte is read exactly once by the whole grid and is fetched with the non-temporal hint; with several row
// blocks on an expert the later ones find the fragment in the L2 and the hint would take that away.
template <int VPL, bool ONCE>
__global__ __launch_bounds__(kDecNW * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void moe_decode_layer_kernel(const DecodeParams p) {
  constexpr int NW = kDecNW, XS = kDecXS, NT = NW * 64;
  typedef Frag<16> FR;
  __shared__ int16_t eid_s[kDecMaxRows];      // expert of flat entry f = t*k + j
  __shared__ float gate_s[kDecMaxRows];       // its gate value
  __shared__ int16_t rowflat_s[kDecMaxRows];  // flat entry of expert-sorted row
  __shared__ int32_t hist_s[kDecMaxExperts];
  __shared__ int32_t offs_s[kDecMaxExperts + 1];  // first expert-sorted row of expert e
  __shared__ int16_t act_s[kDecMaxExperts];       // a -> expert id, active experts in ascending order
  __shared__ int32_t bpre_s[kDecMaxExperts + 1];  // a -> 16-row blocks of the active experts before a
  __shared__ int32_t misc_s[4];                   // [0] number of active experts
  __shared__ DecUnit tab_s[kDecMaxUnits + kDecRing];
  // partial sums of a unit: [unit parity][wave][half][lane] (a lane's two quads 1 KiB apart: 16-byte accesses of
  // neighbouring lanes are then contiguous, without bank conflicts)
  __shared__ f32x4_t red_s[2][NW][2][64];
  __shared__ __attribute__((aligned(16))) float bias_s[kDecMaxUnits][32];  // bias of a unit's 32 columns
  __shared__ u32x4_t xst_s[NW][4][64];  // per wave: one K-stage of a row block's activations on its way into MFMA order

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, kg = lane >> 4;
  const int T = p.T, E = p.E, k = p.k, R = T * k;
  const int G = (int)gridDim.x;

  DEC_STAMP(0);
  // ---- 1. routing, by every workgroup for itself ----------------------------------------------------------
  // Sixteen lanes (one DPP row) own a token, four tokens per wave at a time; lane l of the row holds the VPL
  // consecutive experts l*VPL .. l*VPL+VPL-1 as order-preserving keys.  A round = the row's largest key still in the
  // running (in-lane maximum, then four DPP steps inside the row) and the LOWEST expert index holding it (same again
  // with a minimum): ties go to the lower expert, as the reference's packed sort key does
  // (topk_details/_topk_forward.py:27-35,61).  No lane leaves its row, so the four tokens cost what one costs.
  // [token word][expert]: bit t of word w = token 32 w + t chose the expert.  (Experts along the rows: in the other order the
  // lanes of the counting pass below, which own neighbouring experts, all met in one LDS bank.)
  int32_t(*mask_s)[kDecMaxExperts] = reinterpret_cast<int32_t(*)[kDecMaxExperts]>(&red_s[0][0][0][0]);
  {
    const int l16 = lane & 15, sub = lane >> 4;
    for (int row0 = 0; row0 < T; row0 += NW * 4) {
      const bool wave_has_rows = row0 + wave * 4 < T;  // (uniform) a wave without tokens stays out of the others' way
      if (!wave_has_rows && row0 > 0) break;
      const int row = row0 + wave * 4 + sub;
      const bool row_ok = row < T;
      uint32_t key[VPL];
      uint32_t ret = 0;  // bit i: key[i] is out of the running
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const int e = l16 * VPL + i;
        float f = 0.f;
        if (row_ok && e < E) {
          const int64_t at = (int64_t)row * p.logits_stride + e;
          f = p.logits_is_bf16 ? bf16_bits_to_f32(static_cast<const uint16_t*>(p.logits)[at]) : static_cast<const float*>(p.logits)[at];
        }
        key[i] = ordered_key(f);
        ret |= (e >= E ? 1u : 0u) << i;
      }
      if (row0 == 0) {  // the masks are cleared while the first logits are on their way (every wave comes through here)
        for (int i = tid; i < kDecMaxExperts * ((T + 31) >> 5); i += NT) (&mask_s[0][0])[i] = 0;
        __syncthreads();
        DEC_STAMP(17);
      }
      if (!wave_has_rows) break;
      if (row0 == 0 && key[0] == 0x12345u) DEC_STAMP(9);  // (never true: makes the stamp below wait for the logits)
      if (row0 == 0) DEC_STAMP(18);
      uint32_t sel_key[2] = {0u, 0u};
      int sel_idx[2] = {0, 0};
      uint32_t key0 = 0;
      row16_topk<VPL>(key, ret, k, l16, sel_key, sel_idx, key0);
      if (row0 == 0) DEC_STAMP(19);
      // softmax over the k kept logits (fp32): z = exp(v - max) / sum
      float outv[2], z[2];
      const float vmax = key_to_float(key0);
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const bool have = l16 + 16 * q < k;
        outv[q] = key_to_float(sel_key[q]);
        z[q] = have ? expf(outv[q] - vmax) : 0.f;
      }
      if (p.apply_softmax) {
        const float sum = row16_sum_f32(z[0] + z[1]);
        outv[0] = z[0] / sum;
        outv[1] = z[1] / sum;
      }
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const int j = l16 + 16 * q;
        if (row_ok && j < k) {
          int e = sel_idx[q];
          e = e < 0 ? 0 : (e < E ? e : E - 1);  // (k <= E: every round finds a column)
          eid_s[row * k + j] = (int16_t)e;
          gate_s[row * k + j] = outv[q];
          atomicOr(&mask_s[row >> 5][e], 1 << (row & 31));
          if (blockIdx.x == 0) {
            if (p.indx_out) p.indx_out[row * k + j] = (int16_t)e;
            if (p.vals_out) p.vals_out[row * k + j] = outv[q];
          }
        }
      }
    }
  }
  __syncthreads();
  DEC_STAMP(1);
  // ---- rows per expert, expert offsets, the list of active experts and their row blocks (wave 0) ----------
  const int tw = (T + 31) >> 5;  // token words in use
  if (wave == 0) {
    constexpr int PER = VPL * 16 / 64;  // experts per lane (the kernel's variant covers VPL * 16 experts)
    int cnt[PER];
    int rows = 0, blks = 0, acts = 0;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = lane * PER + i;
      int c = 0;
      if (e < E)
        for (int w = 0; w < tw; ++w) c += __builtin_popcount((uint32_t)mask_s[w][e]);
      cnt[i] = c;
      rows += c;
      blks += (c + 15) >> 4;
      acts += c > 0 ? 1 : 0;
    }
    const int prow = wave_scan_i32(rows), pblk = wave_scan_i32(blks), pact = wave_scan_i32(acts);  // inclusive, over the lanes
    int r0 = prow - rows, b0 = pblk - blks, a0 = pact - acts;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = lane * PER + i;
      if (e < E) {
        hist_s[e] = cnt[i];
        offs_s[e] = r0;
        if (cnt[i] > 0) {
          act_s[a0] = (int16_t)e;
          bpre_s[a0] = b0;
          ++a0;
        }
        r0 += cnt[i];
        b0 += (cnt[i] + 15) >> 4;
      }
    }
    if (lane == 63) {
      offs_s[E] = prow;
      bpre_s[pact] = pblk;
      misc_s[0] = pact;
    }
  }
  __syncthreads();
  // ---- expert-sorted row order (stable): entry (t, j) of expert e goes behind the entries of e from earlier tokens ----
  for (int f = tid; f < R; f += NT) {
    const int e = eid_s[f], t = f / k;
    int rank = 0;
    for (int w = 0; w < (t >> 5); ++w) rank += __builtin_popcount((uint32_t)mask_s[w][e]);
    rank += __builtin_popcount((uint32_t)mask_s[t >> 5][e] & ((1u << (t & 31)) - 1u));
    rowflat_s[offs_s[e] + rank] = (int16_t)f;
  }
  const int A = misc_s[0];
  const int nblk = bpre_s[A];
  // ---- 2. this workgroup's share of the unit lists ---------------------------------------------------------
  // unit uu of a list = (row block uu / nfr, fragment uu % nfr): a workgroup's run stays on one row block, whose
  // activation rows its waves keep in registers.  The row blocks are cut into two halves and every workgroup works
  // through four runs: GEMM 1 of the first half, GEMM 1 of the second, GEMM 2 of the first, GEMM 2 of the second.
  // When a workgroup reaches a GEMM-2 run, the rows of h it needs were finished (by all workgroups) a whole run
  // earlier, so the hand-over between the GEMMs costs no waiting.
  const int bh = (nblk + 1) >> 1;  // row blocks of the first half
  // (32-bit arithmetic: nblk <= 272 and nfr1 + nfr2 <= 288, so G * (U1 + U2) stays below 2^25; a 64-bit division is
  // a hundred instructions, and a dozen of them stood between the routing and the first weight request)
  const int U1 = nblk * p.nfr1, U2 = nblk * p.nfr2;
  const int L0 = bh * p.nfr1, L1 = U1 - L0, L2 = bh * p.nfr2, L3 = U2 - L2;
  const int wg = blockIdx.x;
  auto udiv = [](int a, int b) -> int { return (int)((uint32_t)a / (uint32_t)b); };
  // Shares.  The four runs are cut as one list: cut i of a run = floor(i * (S + L) / G) - floor(i * S / G), S = the
  // units of the runs in front of it, L its own, so that what a workgroup has got from the runs so far is
  // floor((i + 1) * S / G) - floor(i * S / G) whatever the remainders were: a workgroup's units of the whole layer
  // differ by at most one from any other's, and so do its units of GEMM 1 (the GEMM-2 runs wait for everybody's
  // GEMM-1 runs).  A unit of either GEMM costs the same, and with a dozen units per workgroup one more in every run is a
  // quarter more work.  The cuts grow with i when L >= 2 G (their increment is at least L / G - 2); a shorter run is cut
  // evenly by itself and the list starts again with it.
  int S = 0;
  auto share = [&](int L, int& cut_b, int& cut_e) {
    if (S != 0 && L < 2 * G) S = 0;
    cut_b = udiv(wg * (S + L), G) - udiv(wg * S, G);
    cut_e = udiv((wg + 1) * (S + L), G) - udiv((wg + 1) * S, G);
    S += L;
  };
  int c0b, c1b, c0e, c1e, c2b, c3b, c2e, c3e;
  share(L0, c0b, c0e);
  share(L1, c1b, c1e);
  share(L2, c2b, c2e);
  share(L3, c3b, c3e);
  const int r0b = c0b, r0e = c0e, r1b = L0 + c1b, r1e = L0 + c1e;
  const int r2b = c2b, r2e = c2e, r3b = L2 + c3b, r3e = L2 + c3e;
  int nr0 = r0e - r0b, nr1 = r1e - r1b, nr2 = r2e - r2b, nr3 = r3e - r3b;
  if (nr0 + nr1 + nr2 + nr3 > kDecMaxUnits) {  // (the host's bound rules this out)
    if (tid == 0) atomicOr(&p.sync[1], 2);
    nr0 = nr0 < kDecMaxUnits ? nr0 : kDecMaxUnits;
    nr1 = nr1 < kDecMaxUnits - nr0 ? nr1 : kDecMaxUnits - nr0;
    nr2 = nr2 < kDecMaxUnits - nr0 - nr1 ? nr2 : kDecMaxUnits - nr0 - nr1;
    nr3 = nr3 < kDecMaxUnits - nr0 - nr1 - nr2 ? nr3 : kDecMaxUnits - nr0 - nr1 - nr2;
  }
  const int n1 = nr0 + nr1, n2 = nr2 + nr3;
  const int n_units = n1 + n2;
  // (no barrier here: the table below is built from the scan's results, like the row order above)
  for (int i = tid; i < n_units + kDecRing; i += NT) {
    DecUnit u;
    if (i >= n_units) {  // what the loads issued during the last units fetch: one fixed block, never used
      u.w = p.w1;
      u.s = p.w1s;
      u.key = -1;
      u.frag = 0;
    } else {
      const bool ph2 = i >= n1;
      const int uu = i < nr0 ? r0b + i : i < n1 ? r1b + (i - nr0) : i < n1 + nr2 ? r2b + (i - n1) : r3b + (i - n1 - nr2);
      const int nfr = ph2 ? p.nfr2 : p.nfr1;
      const int nst = ph2 ? p.nst2 : p.nst1;
      const int B = udiv(uu, nfr), F = uu - B * nfr;
      int lo = 0, hi = A;  // last a with bpre[a] <= B
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (bpre_s[mid] <= B) lo = mid; else hi = mid;
      }
      const int a = lo, rb = B - bpre_s[a];
      const int e = act_s[a];
      u.w = (ph2 ? p.w2 + (int64_t)e * p.w2_stride_e : p.w1 + (int64_t)e * p.w1_stride_e) + (int64_t)F * nst * 2048;
      u.s = (ph2 ? p.w2s + (int64_t)e * p.w2s_stride_e : p.w1s + (int64_t)e * p.w1s_stride_e) + (int64_t)F * nst * 128;
      u.key = ((ph2 ? 2 : 1) << 24) | (a << 8) | rb;
      u.frag = F;
    }
    tab_s[i] = u;
  }
  __syncthreads();  // (the token masks are dead from here on: their memory becomes the reduction buffers)
  DEC_STAMP(2);

  // ---- 3. the stream ----------------------------------------------------------------------------------------
  // lane (lr, kg): weight columns g*16 + lr of the fragment, k-block kg (32 k = 16 packed bytes) of every stage;
  // this wave's stages of a unit are wave*XS + j
  const uint32_t wlane = (uint32_t)((kg & 1) * 1024 + ((kg >> 1) * 32 + lr) * 16);
  const uint32_t slane = (uint32_t)(lr * 4);
  // weight registers: RD sets of XS stages; unit i lives in set i % RD and, stage by stage as it is consumed, is
  // replaced by unit i + RD.  A wave's requests are answered in order, one unit per unit time, so a block must be
  // requested RD unit times before it is used: with a loaded memory latency of about 4 us, two sets bound a unit at
  // 2 us (what was measured), three at 1.3 us, which is below what HBM delivers (19 KiB per wave on its way).
  constexpr int RD = kDecRing;
  u32x4_t wr[RD][XS][2];
  uint32_t sr[RD][XS][2];
  u32x4_t xr[XS][4];
  auto load_w = [&](auto h_c, int j, const DecUnit& u, int nst) __attribute__((always_inline)) {
    constexpr int H = decltype(h_c)::value;
    int s = wave * XS + j;
    s = s < nst ? s : nst - 1;  // stages past the last re-read it (no branch around a load: the compiler's wait counts
                                // stay exact only in straight-line code); their scales are taken as zero when they are used
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      // (global address space spelled out: the pointers come out of the LDS table, the compiler takes them for generic
      // ones, and with FLAT loads in flight every wait for memory on this target is a wait for ALL of it, i.e. the ring
      // of weight blocks would be drained at the head of every unit)
      const auto* wp = (const __attribute__((address_space(1))) u32x4_t*)(u.w + (int64_t)s * 2048 + g * 256 + wlane);
      const auto* sp = (const __attribute__((address_space(1))) uint32_t*)(u.s + (int64_t)s * 128 + g * 64 + slane);
      if constexpr (ONCE) {
        wr[H][j][g] = __builtin_nontemporal_load(wp);
        sr[H][j][g] = __builtin_nontemporal_load(sp);
      } else {
        wr[H][j][g] = *wp;
        sr[H][j][g] = *sp;
      }
    }
  };
  auto unit_nst = [&](const DecUnit& u) __attribute__((always_inline)) -> int { return (u.key >> 24) == 2 ? p.nst2 : p.nst1; };
  const __amdgpu_buffer_rsrc_t hrsrc = __builtin_amdgcn_make_buffer_rsrc(p.h, 0, (uint32_t)((int64_t)R * p.K2 * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t yrsrc = __builtin_amdgcn_make_buffer_rsrc(p.y, 0, (uint32_t)((int64_t)R * p.N2 * 2), 0x00020000);
  const float nalpha_log2e = -p.alpha * 1.4426950408889634f;
  const float limit = p.has_limit ? p.limit : INFINITY;

  // table entries are the same for every lane: keep them in scalar registers
  auto uniform_unit = [&](int i) __attribute__((always_inline)) -> DecUnit {
    const DecUnit v = tab_s[i];
    const uint64_t w = (uint64_t)v.w, sc = (uint64_t)v.s;
    DecUnit u;
    u.w = (const uint8_t*)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(w >> 32)) << 32) | (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)w));
    u.s = (const uint8_t*)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(sc >> 32)) << 32) | (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)sc));
    u.key = __builtin_amdgcn_readfirstlane(v.key);
    u.frag = __builtin_amdgcn_readfirstlane(v.frag);
    return u;
  };
  // counts GEMM-1 units [from, to) of this workgroup in at their row blocks' counters (unit u belongs to block u / nfr1)
  auto signal_blocks = [&](int ub, int ue) __attribute__((always_inline)) {
    if (ue > ub) {
      const int b_first = udiv(ub, p.nfr1), b_last = udiv(ue - 1, p.nfr1);
      for (int b = b_first + tid; b <= b_last; b += NT) {
        const int lo = b * p.nfr1, hi = lo + p.nfr1;
        const int from = lo > ub ? lo : ub, to = hi < ue ? hi : ue;
        __hip_atomic_fetch_add(&p.sync[2 + b * kDecBlockStride], to - from, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  };
  // This wave's K-slice of a row block's activation rows: x through the expert-sorted order for GEMM 1, h for GEMM 2.
  // The MFMA wants row lr's k-block kg in lane (lr, kg): loaded that way, the sixteen lanes that one pass of a load
  // serves touch sixteen rows, i.e. sixteen cache lines for 16 bytes each.  So the rows are loaded four lanes to a row
  // (lane = row * 4 + chunk: 64 contiguous bytes per row and instruction, rows past the block's last dropped, not
  // repeated) and turned into MFMA order through a 4 KiB buffer of the wave's own in LDS, one K-stage at a time
  // (LDS operations of a wave execute in order; 16-byte chunks swizzled by the row so that neither side conflicts).
  const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.x), 0, p.x_bytes, 0x00020000);
  auto x_request = [&](auto ph_c, const DecUnit& u) __attribute__((always_inline)) {
    constexpr int ph = decltype(ph_c)::value;  // 1: rows of x, 2: rows of h
    const int a = (u.key >> 8) & 0xFFFF, rb = u.key & 0xFF;
    const int e = act_s[a];
    const int cnt = hist_s[e];
    const int row0 = offs_s[e] + rb * 16;
    const int rows = cnt - rb * 16 < 16 ? cnt - rb * 16 : 16;
    const int r = lane >> 2, c = lane & 3;
    const bool valid = r < rows;
    const int K = ph == 2 ? p.K2 : p.K1;
    // first k of this lane in its wave's slice (opaque: otherwise the twelve addresses below are computed once, ahead
    // of the loop, and parked in scratch memory, which turns every reload into a chain of dependent memory round trips)
    int kb = wave * (XS * 128) + c * 8;
    asm volatile("" : "+v"(kb));
    uint32_t base;
    if constexpr (ph == 2) {
      base = (uint32_t)(row0 + r) * (uint32_t)(p.K2 * 2);
    } else {
      const int token = rowflat_s[row0 + (valid ? r : 0)] / k;
      base = (uint32_t)token * (uint32_t)(p.x_stride * 2);
    }
#pragma unroll
    for (int j = 0; j < XS; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int k0 = kb + j * 128 + q * 32;
        // past K the weights are zero (padding) or their scales are zeroed (stages past the last): zeros will do
        const uint32_t off = (valid && k0 < K) ? base + (uint32_t)k0 * 2u : kDroppedStore;
        if constexpr (ph == 2)
          xr[j][q] = __builtin_amdgcn_raw_buffer_load_b128(hrsrc, off, 0, kThrough);
        else
          xr[j][q] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, off, 0, 0);
      }
  };
  auto x_settle = [&]() __attribute__((always_inline)) {
    const int r = lane >> 2, c = lane & 3;
    const int wpos = r * 4 + (c ^ ((r >> 2) & 3));
#pragma unroll
    for (int j = 0; j < XS; ++j) {
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int q = 0; q < 4; ++q) xst_s[wave][q][wpos] = xr[j][q];
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int t = 0; t < 4; ++t) xr[j][t] = xst_s[wave][kg][lr * 4 + (t ^ ((lr >> 2) & 3))];
    }
  };
  int cur_key = 0;
  if (n_units > 0) {
    // the first unit's activation slice is requested in front of the weight blocks (a wave's requests are answered in
    // order, and the three units of weight blocks primed below keep the memory system busy for microseconds)
    const DecUnit first = uniform_unit(0);
    const bool x_first = (first.key >> 24) == 1;
    if (x_first) {
      x_request(std::integral_constant<int, 1>{}, first);
      cur_key = first.key;
    }
    static_for<0, RD>([&](auto h_c) __attribute__((always_inline)) {
      const DecUnit u = uniform_unit(decltype(h_c)::value);
#pragma unroll
      for (int j = 0; j < XS; ++j) load_w(h_c, j, u, unit_nst(u));
    });
    // (here, in straight-line code behind the requests, the wait in front of the LDS writes counts the weight blocks
    // out: behind the bias loops below it would be a wait for everything requested so far)
    if (x_first) x_settle();
  }
  // The biases of this workgroup's units (32 columns each) go to LDS once: requested behind the first weight blocks,
  // written in front of the first unit's barrier.  Four values per thread cover 64 units; more take another round.
  constexpr int BPT = 4;
  uint32_t bias_raw[BPT];
  auto bias_fetch = [&](int first_unit) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < BPT; ++q) {
      const int idx = first_unit * 32 + q * NT + tid, ui = idx >> 5, c = idx & 31;
      bias_raw[q] = 0u;
      if (ui < n_units) {
        const DecUnit u = tab_s[ui];
        const bool ph2 = (u.key >> 24) == 2;
        const void* bp = ph2 ? p.b2 : p.b1;
        const int n = u.frag * 32 + c;
        if (bp && n < (ph2 ? p.N2 : p.N1)) {
          const int64_t at = (int64_t)act_s[(u.key >> 8) & 0xFFFF] * (ph2 ? p.b2_stride_e : p.b1_stride_e) + n;
          // (raw bits: anything computed from the value here would wait for it, behind the weight blocks just requested)
          bias_raw[q] = (ph2 ? p.b2_is_f32 : p.b1_is_f32) ? static_cast<const uint32_t*>(bp)[at] : (uint32_t)static_cast<const uint16_t*>(bp)[at];
        }
      }
    }
  };
  auto bias_park = [&](int first_unit) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < BPT; ++q) {
      const int idx = first_unit * 32 + q * NT + tid;
      const int ui = idx >> 5;
      if (ui < n_units) {
        const bool f32 = (tab_s[ui].key >> 24) == 2 ? p.b2_is_f32 : p.b1_is_f32;
        (&bias_s[0][0])[idx] = bits_f32(f32 ? bias_raw[q] : bias_raw[q] << 16);
      }
    }
  };
  constexpr int kBiasRound = BPT * NT / 32;  // units per round
  for (int u0 = kBiasRound; u0 < n_units; u0 += kBiasRound) {  // (more than 64 units: the later rounds up front)
    bias_fetch(u0);
    bias_park(u0);
  }
  DEC_STAMP(12);
  bias_fetch(0);
  DEC_STAMP(13);
  // A finished GEMM-1 run is counted in without draining the wave's memory queue.  A wave's loads and stores complete
  // in issue order.  The epilogue of a run's last unit stores its rows of h right behind that unit's barrier; the
  // next unit opens another row block (or the other GEMM), so EVERY wave starts it by fetching new activation rows
  // and consumes them in its K loop.  Behind that unit's barrier all stores of the finished run have therefore
  // reached memory, and the run is counted in there.  (A wait that comes earlier than that, possible only for a
  // workgroup with next to no units, drains the queue and counts in first: a workgroup must never wait for rows
  // that it has not counted in itself.)
  bool signalled0 = nr0 == 0, signalled = n1 == 0;
  auto unit_body = [&](auto h_c, int i) __attribute__((always_inline)) {
    constexpr int H = decltype(h_c)::value;
    const DecUnit cur = uniform_unit(i);
    const DecUnit nxt = uniform_unit(i + RD);  // the unit that takes over this set of weight registers
    const int ph = cur.key >> 24, a = (cur.key >> 8) & 0xFFFF, rb = cur.key & 0xFF;
    const int e = act_s[a];
    const int cnt = hist_s[e];
    const int row0 = offs_s[e] + rb * 16;                       // first expert-sorted row of the block
    const int rows = cnt - rb * 16 < 16 ? cnt - rb * 16 : 16;  // valid rows of the block
    if (i == 1) DEC_STAMP(3);
    if (i == n1) DEC_STAMP(4);
    if (cur.key != cur_key) {
      cur_key = cur.key;
      // ---- a new (expert, row block): this wave's K-slice of its activation rows goes into registers ----
      if (ph == 2) {
        const int blk = bpre_s[a] + rb;  // a block of the first half was computed by run 0 alone
        if (!signalled0 || (blk >= bh && !signalled)) {  // (uniform) see above: count in what this workgroup itself still owes
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          __syncthreads();
          if (!signalled0) signal_blocks(r0b, r0b + nr0);
          if (!signalled) signal_blocks(r1b, r1b + nr1);
          signalled0 = signalled = true;
        }
        // the block's rows of h are complete when all nfr1 GEMM-1 units of the block have been counted in
        if (tid == 0) {
          int spins = 0;
          // (polled gently, and every block's counter in a cache line of its own: a few hundred workgroups polling
          // one line at full speed slow down every stream that crosses that memory channel)
          while (__hip_atomic_load(&p.sync[2 + blk * kDecBlockStride], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < p.nfr1) {
            __builtin_amdgcn_s_sleep(16);
            if (++spins > p.spin_limit) {
              atomicOr(&p.sync[1], 1);
              break;
            }
          }
        }
        __syncthreads();
        if (i == n1) DEC_STAMP(5);
        x_request(std::integral_constant<int, 2>{}, cur);
      } else {
        x_request(std::integral_constant<int, 1>{}, cur);
      }
      x_settle();
    }
    if (i == 0) DEC_STAMP(14);
    const bool leader = (i % NW) == wave;
    const int F = cur.frag;
    // ---- this wave's K-slice of the unit; the next unit's blocks follow into the slots as they fall free ----
    typename FR::acc_t acc[2];
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[g][c] = 0.f;
    const int nst_next = unit_nst(nxt);
    const int nst_cur = ph == 2 ? p.nst2 : p.nst1;
#pragma unroll
    for (int j = 0; j < XS; ++j) {
      const uint32_t live = wave * XS + j < nst_cur ? 0xFFu : 0u;  // (uniform) a stage past the last contributes nothing
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        bf16x8_t wf[2];
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          const u32x4_t v = wr[H][j][g];
          const uint32_t raw = t == 0 ? v.x : t == 1 ? v.y : t == 2 ? v.z : v.w;
          wf[g] = dequant8(raw, bits_f32(((sr[H][j][g] >> (8 * kg)) & live) << 23));
        }
        const bf16x8_t xf = __builtin_bit_cast(bf16x8_t, xr[j][t]);
#pragma unroll
        for (int g = 0; g < 2; ++g) acc[g] = FR::mma(wf[g], xf, acc[g]);
      }
      load_w(h_c, j, nxt, nst_next);
    }
    // ---- the slices meet in LDS; the leader sums them in slice order and runs the epilogue ----
    if (i == 0) DEC_STAMP(15);
    DEC_UNIT_STAMP(i);
    if (i == 0) bias_park(0);
    {
      red_s[i & 1][wave][0][lane] = acc[0];
      red_s[i & 1][wave][1][lane] = acc[1];
    }
    __syncthreads();
    if (i == 0) DEC_STAMP(16);
    if (i == nr0 && !signalled0) {  // the first unit behind run 0 (it exists and opened a new row block)
      signalled0 = true;
      signal_blocks(r0b, r0b + nr0);
    }
    if (i == n1 && !signalled) {  // the first GEMM-2 unit
      signalled = true;
      signal_blocks(r1b, r1b + nr1);
    }
    if (leader) {
      const int row_c = lr < rows ? lr : rows - 1;
      const int flat = rowflat_s[row0 + row_c];
      const float gam = gate_s[flat];
      const f32x4_t bias_lo = *reinterpret_cast<const f32x4_t*>(&bias_s[i][kg * 4]);
      const f32x4_t bias_hi = *reinterpret_cast<const f32x4_t*>(&bias_s[i][16 + kg * 4]);
      f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int q = 0; q < NW; ++q) {
        s0 += red_s[i & 1][q][0][lane];
        s1 += red_s[i & 1][q][1][lane];
      }
      const bool row_ok = lr < rows;
      if (ph == 1) {
        // bias, swiglu over the interleaved (gate, linear) pairs, bf16, row (row0 + lr) of h
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          const f32x4_t s = (g == 0 ? s0 : s1) + (g == 0 ? bias_lo : bias_hi);
          const int n0 = F * 32 + g * 16 + kg * 4;
          const float o0 = swiglu_f(s[0], s[1], nalpha_log2e, limit);
          const float o1 = swiglu_f(s[2], s[3], nalpha_log2e, limit);
          const uint32_t off = (row_ok && n0 < p.N1) ? (uint32_t)(row0 + lr) * (uint32_t)(p.K2 * 2) + (uint32_t)(n0 / 2) * 2u : kDroppedStore;
          __builtin_amdgcn_raw_buffer_store_b32(pack_bf16x2(o0, o1), hrsrc, off, 0, kThrough);
        }
      } else {
        // bias, gate weight, bf16, flat row t*k + j of y
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          const f32x4_t s = (g == 0 ? s0 : s1) + (g == 0 ? bias_lo : bias_hi);
          const int n0 = F * 32 + g * 16 + kg * 4;
          const u32x2_t w = {pack_bf16x2(s[0] * gam, s[1] * gam), pack_bf16x2(s[2] * gam, s[3] * gam)};
          const uint32_t off = (row_ok && n0 < p.N2) ? (uint32_t)flat * (uint32_t)(p.N2 * 2) + (uint32_t)n0 * 2u : kDroppedStore;
          __builtin_amdgcn_raw_buffer_store_b64(w, yrsrc, off, 0, kThrough);
        }
      }
    }
  };
  // Whole rounds of RD units run without a test between the units: with one, the compiler has to allow for a round
  // that skips its later units and comes back to the first, i.e. for weight blocks that nothing younger follows, and
  // its waits then drain the wave's memory queue once per round.
  int i_unit = 0;
  for (; i_unit + RD <= n_units; i_unit += RD)
    static_for<0, RD>([&](auto h_c) __attribute__((always_inline)) { unit_body(h_c, i_unit + decltype(h_c)::value); });
  static_for<0, RD - 1>([&](auto h_c) __attribute__((always_inline)) {
    if (i_unit + decltype(h_c)::value < n_units) unit_body(h_c, i_unit + decltype(h_c)::value);
  });
  DEC_STAMP(6);
  // ---- 4./5. hand-over of whatever is still to be counted in, then the combine of this workgroup's rows of y ----
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (!signalled0) signal_blocks(r0b, r0b + nr0);
  if (!signalled) signal_blocks(r1b, r1b + nr1);
  DEC_STAMP(7);
  int32_t* arrivals = p.sync + 2 + kDecBlockWords;
  const bool out_vec = (p.out_stride & 7) == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0;
  for (int it0 = 0; it0 < n2 * 64; it0 += NT) {
    // item = (unit, row of its block, group of 8 columns): the group-0 thread counts the row in and tells the other three
    const int it = it0 + tid;
    int seen = -1, token = 0, F = 0;
    if (it < n2 * 64) {
      const DecUnit u = tab_s[n1 + (it >> 6)];
      const int r = (it >> 2) & 15;
      const int a = (u.key >> 8) & 0xFFFF, rb = u.key & 0xFF;
      const int e = act_s[a];
      F = u.frag;
      if (rb * 16 + r < hist_s[e]) {
        token = rowflat_s[offs_s[e] + rb * 16 + r] / k;
        if ((it & 3) == 0) seen = __hip_atomic_fetch_add(&arrivals[token * p.nfr2 + F], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    seen = __shfl(seen, lane & ~3);
    const int n0 = F * 32 + (it & 3) * 8;
    const bool sum_it = seen == k - 1 && n0 < p.N2;
    // all k rows of (token, fragment) are in memory: fp32 sum in j order, bf16 result
    const bool full = n0 + 8 <= p.N2;  // else four columns (N2 is a multiple of 4... of 8 here)
    float sum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j0 = 0; j0 < k; j0 += 4) {
      u32x4_t v[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t off = (sum_it && j0 + q < k) ? (uint32_t)(token * k + j0 + q) * (uint32_t)(p.N2 * 2) + (uint32_t)n0 * 2u : kDroppedStore;
        v[q] = __builtin_amdgcn_raw_buffer_load_b128(yrsrc, off, 0, kThrough);  // dropped offsets read zero
      }
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          sum[2 * c] += bits_f32(v[q][c] << 16);
          sum[2 * c + 1] += bits_f32(v[q][c] & 0xFFFF0000u);
        }
    }
    if (sum_it) {
      uint16_t* o = p.out + (int64_t)token * p.out_stride + n0;
      if (full && out_vec) {
        *reinterpret_cast<u32x4_t*>(o) = u32x4_t{pack_bf16x2(sum[0], sum[1]), pack_bf16x2(sum[2], sum[3]), pack_bf16x2(sum[4], sum[5]), pack_bf16x2(sum[6], sum[7])};
      } else {
        const int nc = p.N2 - n0 < 8 ? p.N2 - n0 : 8;
        for (int c = 0; c < nc; ++c) o[c] = f32_to_bf16_bits(sum[c]);
      }
    }
  }
  // ---- 6. the last workgroup to finish clears the counters for the next launch ----
  __syncthreads();
  DEC_STAMP(8);
#ifdef TK_DEC_STAMPS
  if (tid == 0) { dec_stamps[blockIdx.x][10] = n1; dec_stamps[blockIdx.x][11] = n2; }
#endif
  if (tid == 0) {
    __threadfence();
    misc_s[1] = atomicAdd(&p.sync[0], 1);
  }
  __syncthreads();
  if (misc_s[1] == G - 1) {
    __threadfence();
    for (int b = tid; b < nblk; b += NT) __hip_atomic_store(&p.sync[2 + b * kDecBlockStride], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (int w = tid; w < T * p.nfr2; w += NT) __hip_atomic_store(&arrivals[w], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid == 0) __hip_atomic_store(&p.sync[0], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// workgroups of the kernel that are resident together on the current device (cached per device and variant)
template <int VPL>
int resident_workgroups() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(moe_decode_layer_kernel<VPL, false>), kDecNW * 64, 0) != hipSuccess || per_cu <= 0)
      return 0;
    per_cu = 1;  // (a wave holds up to two units of weight blocks in its registers: one workgroup fills a CU)
    n = per_cu * device_cu_count();
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

}  // namespace
}  // namespace tk

using namespace tk;

#ifdef TK_DEC_STAMPS
extern "C" int32_t tk_debug_dec_stamps(long long* host_out) {
  return hipMemcpyFromSymbol(host_out, HIP_SYMBOL(dec_stamps), sizeof(long long) * 1024 * 20) == hipSuccess ? 0 : 3;
}
#endif

extern "C" int64_t tk_moe_decode_layer_workspace_bytes(int32_t n_tokens, int32_t k, int32_t n_experts, int32_t d_ff, int32_t d_model) {
  if (n_tokens <= 0 || k <= 0 || n_experts <= 0 || d_ff <= 0 || d_model <= 0) return 0;
  const int64_t R = (int64_t)n_tokens * k;
  const int64_t hb = (R * d_ff * 2 + 255) / 256 * 256, yb = (R * d_model * 2 + 255) / 256 * 256;
  return hb + yb + (2 + (int64_t)kDecBlockWords + (int64_t)n_tokens * cdiv(d_model, 32)) * 4;
}

extern "C" int32_t tk_moe_decode_layer(const tk_decode_layer_desc* d, tk_stream_t stream) {
  if (!d) return fail(TK_ERR_INVALID, "tk_moe_decode_layer: null descriptor");
  const int T = d->n_tokens, E = d->n_experts, k = d->k;
  if (T < 0 || E <= 0 || k <= 0 || d->d_model <= 0 || d->d_ff <= 0) return fail(TK_ERR_INVALID, "tk_moe_decode_layer: bad sizes T=%d E=%d k=%d d_model=%d d_ff=%d", T, E, k, d->d_model, d->d_ff);
  if (T == 0) return TK_OK;
  if (k > E || k > 32) return fail(TK_ERR_INVALID, "tk_moe_decode_layer: k=%d must be <= min(32, E)", k);
  if ((int64_t)T * k > kDecMaxRows) return fail(TK_ERR_UNSUPPORTED, "tk_moe_decode_layer: at most %d routed rows (got %d x %d); larger batches take tk_route + tk_moe_gemm", kDecMaxRows, T, k);
  if (E > kDecMaxExperts) return fail(TK_ERR_UNSUPPORTED, "tk_moe_decode_layer: at most %d experts (got %d)", kDecMaxExperts, E);
  const int kmax = kDecNW * kDecXS * 128;
  if (d->d_model > kmax || d->d_ff > kmax) return fail(TK_ERR_UNSUPPORTED, "tk_moe_decode_layer: d_model and d_ff must be <= %d (got %d, %d)", kmax, d->d_model, d->d_ff);
  if (d->d_model % 8 || d->d_ff % 8) return fail(TK_ERR_UNSUPPORTED, "tk_moe_decode_layer: d_model and d_ff must be multiples of 8 (got %d, %d)", d->d_model, d->d_ff);
  if (!d->x || !d->logits || !d->w1 || !d->w1_mx_scale || !d->w2 || !d->w2_mx_scale || !d->out || !d->workspace) return fail(TK_ERR_INVALID, "tk_moe_decode_layer: null operand");
  if (d->logits_dtype != TK_F32 && d->logits_dtype != TK_BF16) return fail(TK_ERR_UNSUPPORTED, "tk_moe_decode_layer: logits must be fp32 or bf16");
  if ((d->b1 && d->b1_dtype != TK_F32 && d->b1_dtype != TK_BF16) || (d->b2 && d->b2_dtype != TK_F32 && d->b2_dtype != TK_BF16)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_decode_layer: biases must be fp32 or bf16");
  if ((reinterpret_cast<uintptr_t>(d->x) & 15) || d->x_stride_m % 8) return fail(TK_ERR_UNSUPPORTED, "tk_moe_decode_layer: activation rows must be 16-byte aligned");
  if ((reinterpret_cast<uintptr_t>(d->workspace) & 255)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_decode_layer: the workspace must be 256-byte aligned");
  for (const void* q : {d->w1, d->w2})
    if (reinterpret_cast<uintptr_t>(q) & 15) return fail(TK_ERR_UNSUPPORTED, "tk_moe_decode_layer: tiled weights must be 16-byte aligned");
  for (const void* q : {d->w1_mx_scale, d->w2_mx_scale})
    if (reinterpret_cast<uintptr_t>(q) & 3) return fail(TK_ERR_UNSUPPORTED, "tk_moe_decode_layer: tiled scales must be 4-byte aligned");
  DecodeParams p;
  p.x = static_cast<const uint8_t*>(d->x);
  p.x_stride = d->x_stride_m;
  {
    const int64_t extent = ((int64_t)(T - 1) * d->x_stride_m + d->d_model) * 2;
    if (d->x_stride_m < d->d_model || extent > 0x7FFFFFFFll) return fail(TK_ERR_UNSUPPORTED, "tk_moe_decode_layer: activation rows must not overlap and must lie within 2 GiB (row stride %lld)", (long long)d->x_stride_m);
    p.x_bytes = (uint32_t)extent;
  }
  p.logits = d->logits;
  p.logits_stride = d->logits_stride_m;
  p.logits_is_bf16 = d->logits_dtype == TK_BF16;
  p.T = T;
  p.E = E;
  p.k = k;
  p.apply_softmax = d->apply_softmax;
  p.K1 = d->d_model;
  p.N1 = 2 * d->d_ff;
  p.K2 = d->d_ff;
  p.N2 = d->d_model;
  p.nst1 = (int)cdiv(p.K1, 128);
  p.nst2 = (int)cdiv(p.K2, 128);
  p.nfr1 = (int)cdiv(p.N1, 32);
  p.nfr2 = (int)cdiv(p.N2, 32);
  if (d->w1_stride_e % 16 || d->w2_stride_e % 16 || d->w1s_stride_e % 4 || d->w2s_stride_e % 4) return fail(TK_ERR_UNSUPPORTED, "tk_moe_decode_layer: expert strides of tiled weights must be multiples of 16 (scales: 4) bytes");
  if (E > 1 && (d->w1_stride_e < (int64_t)p.nfr1 * p.nst1 * 2048 || d->w1s_stride_e < (int64_t)p.nfr1 * p.nst1 * 128 ||
                d->w2_stride_e < (int64_t)p.nfr2 * p.nst2 * 2048 || d->w2s_stride_e < (int64_t)p.nfr2 * p.nst2 * 128))
    return fail(TK_ERR_INVALID, "tk_moe_decode_layer: expert stride smaller than one tiled expert");
  p.w1 = static_cast<const uint8_t*>(d->w1);
  p.w1s = static_cast<const uint8_t*>(d->w1_mx_scale);
  p.w1_stride_e = d->w1_stride_e;
  p.w1s_stride_e = d->w1s_stride_e;
  p.b1 = d->b1;
  p.b1_stride_e = d->b1_stride_e;
  p.b1_is_f32 = d->b1_dtype == TK_F32;
  p.w2 = static_cast<const uint8_t*>(d->w2);
  p.w2s = static_cast<const uint8_t*>(d->w2_mx_scale);
  p.w2_stride_e = d->w2_stride_e;
  p.w2s_stride_e = d->w2s_stride_e;
  p.b2 = d->b2;
  p.b2_stride_e = d->b2_stride_e;
  p.b2_is_f32 = d->b2_dtype == TK_F32;
  p.alpha = d->act_alpha;
  p.limit = d->act_limit;
  p.has_limit = d->act_has_limit;
  const int64_t R = (int64_t)T * k;
  const int64_t hb = (R * p.K2 * 2 + 255) / 256 * 256, yb = (R * p.N2 * 2 + 255) / 256 * 256;
  uint8_t* ws = static_cast<uint8_t*>(d->workspace);
  p.h = reinterpret_cast<uint16_t*>(ws);
  p.y = reinterpret_cast<uint16_t*>(ws + hb);
  p.sync = reinterpret_cast<int32_t*>(ws + hb + yb);
  p.out = static_cast<uint16_t*>(d->out);
  p.out_stride = d->out_stride_m;
  p.indx_out = static_cast<int16_t*>(d->indx_out);
  p.vals_out = d->vals_out;
  p.spin_limit = d->spin_limit > 0 ? d->spin_limit : (1 << 22);
  const bool small_e = E <= 128;
  int grid = small_e ? resident_workgroups<8>() : resident_workgroups<kDecMaxExperts / 16>();
  if (grid <= 0) return fail(TK_ERR_LAUNCH, "tk_moe_decode_layer: cannot determine how many workgroups are resident together");
  // units of one workgroup: at most min(E, R) + R / 16 row blocks, each with nfr1 + nfr2 fragments, dealt evenly (+1 per run)
  const int64_t max_blocks = (R < E ? R : E) + R / 16;
  if (max_blocks * (p.nfr1 + p.nfr2) / grid + 4 > kDecMaxUnits)
    return fail(TK_ERR_UNSUPPORTED, "tk_moe_decode_layer: %lld row blocks x %d fragments over %d workgroups exceed the kernel's unit table", (long long)max_blocks, p.nfr1 + p.nfr2, grid);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool once = T <= 16;  // at most 16 rows, i.e. one row block, per expert: measured 43.0 -> 41.5 us at T = 4, 63.9 -> 61.1 at 16
                              // (gpt-oss shape), and 102 -> 107 us at T = 64 with skewed routing, hence the switch
  const dim3 g((unsigned)grid), b(kDecNW * 64);
  if (small_e) {
    if (once)
      hipLaunchKernelGGL((moe_decode_layer_kernel<8, true>), g, b, 0, st, p);
    else
      hipLaunchKernelGGL((moe_decode_layer_kernel<8, false>), g, b, 0, st, p);
  } else {
    if (once)
      hipLaunchKernelGGL((moe_decode_layer_kernel<kDecMaxExperts / 16, true>), g, b, 0, st, p);
    else
      hipLaunchKernelGGL((moe_decode_layer_kernel<kDecMaxExperts / 16, false>), g, b, 0, st, p);
  }
  return check_launch("moe_decode_layer_kernel");
}
