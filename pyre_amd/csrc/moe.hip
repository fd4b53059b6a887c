// MoE FFN block: router logits -> softmax top-k (inside the gate/up launch) -> grouped expert GEMV over only the
// selected experts.
// Follows ffn / routed (f32 branch) of the reference, src/model/qwen4exp_gguf.rs:1675-1684, 1721-1732, 1754-1793,
// and top_k / soft_top / nan_clean, :3121-3139.  All experts are resident in HBM, so there is no host split.
#include "formats.h"
#include "digits.h"
#include "gemm_m.h"
PYRE_TS_DECL(moe_ts) PYRE_TS_EXPORT(moe_ts, pyre_debug_ts_moe)

// ---- router: top-k (ties -> lower index), softmax over the chosen k in ascending expert id -----------------------------
// Runs inside every gate/up workgroup of a routed entry (all of them need the expert id before they can touch a
// weight, and a separate launch would cost more than redoing this small selection everywhere).
// Thread e sums logit e's K slices (in slice order) into shared memory.  The selection is a tournament: every wave
// of 64 logits takes its own k largest (k rounds of: the wave's largest key out of six DPP maximum steps, its lowest lane
// -- the lowest index -- from a ballot, that lane retires its key), the waves' candidates meet in shared memory, each
// candidate counts the candidates that beat it (larger key, or equal key and lower index) and the k that are beaten by
// fewer than k others are the choice.  Leaves the chosen ids (ascending) in s_idx[0..k) and their logits in s_val[0..k).
struct RouteLds { float lv[1024]; float r_val[32]; float s_val[32]; int s_idx[32]; float s_w[32]; uint64_t cand[512]; uint64_t win[32]; };
#ifdef PYRE_PHASE_TS
#define ROUTE_TS_PARAM , unsigned long long* rts_
#define ROUTE_TS_ARG , ts_
#define ROUTE_TS(k) rts_[k] = wall_clock64()
#else
#define ROUTE_TS_PARAM
#define ROUTE_TS_ARG
#define ROUTE_TS(k)
#endif
// A logit becomes a 32-bit key whose unsigned order is the logits' order (0 = no candidate).
__device__ __forceinline__ uint32_t route_key(float v) {
  uint32_t u = __float_as_uint(v + 0.0f);          // -0 counts as +0, as in a float comparison
  return u ^ ((u & 0x80000000u) ? 0xFFFFFFFFu : 0x80000000u);
}
__device__ __forceinline__ float route_key_value(uint32_t u) { return __uint_as_float(u ^ ((u & 0x80000000u) ? 0x80000000u : 0xFFFFFFFFu)); }
template <int CTRL> __device__ __forceinline__ uint32_t route_dpp(uint32_t m) {          // lanes without a source see 0, the maximum's identity: the move folds into the v_max
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, CTRL, 0xf, 0xf, true);
}
__device__ __forceinline__ uint32_t route_wave_max(uint32_t m) {          // idempotent, so the row broadcasts need no row masks
  m = max(m, route_dpp<0x111>(m)); m = max(m, route_dpp<0x112>(m)); m = max(m, route_dpp<0x114>(m)); m = max(m, route_dpp<0x118>(m));      // row_shr 1, 2, 4, 8: lane 15 of a row holds the row's
  m = max(m, route_dpp<0x142>(m)); m = max(m, route_dpp<0x143>(m));          // row_bcast 15, 31: lane 63 holds the wave's
  return (uint32_t)__builtin_amdgcn_readlane((int)m, 63);
}
// called by the whole workgroup (at least n_exp threads, a multiple of 64), after lv[] is complete
__device__ __forceinline__ void route_select(int n_exp, int k, RouteLds& L) {
  const int e = threadIdx.x, lane = e & 63, wave = e >> 6, nwv = (n_exp + 63) >> 6;
  if (wave < nwv) {
    uint32_t key = e < n_exp ? route_key(L.lv[e]) : 0u;
    uint32_t ck = 0u, cl = 0u;          // lane r keeps the wave's r-th candidate
    for (int round = 0; round < k; ++round) {
      const uint32_t wm = route_wave_max(key);
      const int ol = __ffsll((unsigned long long)__ballot(key == wm)) - 1;          // the lowest lane that holds it = the lowest index
      ck = lane == round ? wm : ck; cl = lane == round ? (uint32_t)ol : cl;
      key = lane == ol ? 0u : key;
    }
    if (lane < k) L.cand[wave * k + lane] = ((uint64_t)ck << 32) | (uint32_t)(0xFFFFFFFFu - ((uint32_t)(wave * 64) + cl));
  }
  lds_barrier();
  // eight neighbouring lanes share a candidate and split the others among them; larger 64-bit word = larger key, or the
  // same key at a lower index: a strict order, so the k winners hold the ranks 0 .. k-1
  const int nc = nwv * k, sub = e & 7;
  for (int i = e >> 3; i < nc; i += (int)(blockDim.x >> 3)) {
    const uint64_t ci = L.cand[i];
    int beaten = 0;
#pragma unroll
    for (int jb = 0; jb < 512; jb += 32) if (jb < nc) {          // (uniform branches: with nc known at compile time every read is issued before the first comparison)
      const int j = jb + sub;
      const uint64_t c0 = L.cand[min(j, 511)], c1 = L.cand[min(j + 8, 511)], c2 = L.cand[min(j + 16, 511)], c3 = L.cand[min(j + 24, 511)];
      beaten += ((j < nc && c0 > ci) ? 1 : 0) + ((j + 8 < nc && c1 > ci) ? 1 : 0) + ((j + 16 < nc && c2 > ci) ? 1 : 0) + ((j + 24 < nc && c3 > ci) ? 1 : 0);
    }
    beaten += __builtin_amdgcn_mov_dpp(beaten, 0xB1, 0xf, 0xf, true);          // quad_perm [1,0,3,2]
    beaten += __builtin_amdgcn_mov_dpp(beaten, 0x4E, 0xf, 0xf, true);          // quad_perm [2,3,0,1]
    beaten += __builtin_amdgcn_mov_dpp(beaten, 0x141, 0xf, 0xf, true);         // row_half_mirror: the other quad of the eight
    if (sub == 0 && (uint32_t)(ci >> 32) != 0u && beaten < k) L.win[beaten] = ci;
  }
  lds_barrier();
  if (wave == 0) {
    const uint64_t w = L.win[min(lane, 31)];
    const uint32_t idx = 0xFFFFFFFFu - (uint32_t)w;
    int pos = 0;
    for (int j = 0; j < k; ++j) { const uint32_t oj = (uint32_t)__builtin_amdgcn_readlane((int)idx, j); pos += oj < idx ? 1 : 0; }
    if (lane < k) { L.s_idx[pos] = (int)idx; L.s_val[pos] = route_key_value((uint32_t)(w >> 32)); }
  }
}
// The logits are given as nsl (<= 64) K-slice sums `sstride` floats apart, added in slice order (nsl == 1: the logits
// themselves); all slices are fetched before the first add, in groups of eight behind launch-uniform branches.
__device__ __forceinline__ void route_topk(const float* __restrict__ logits, int nsl, int sstride, int n_exp, int k, RouteLds& L ROUTE_TS_PARAM) {
  const int e = threadIdx.x;
  if (e < n_exp) {
    float sv[64];
#pragma unroll
    for (int q = 0; q < 64; ++q) sv[q] = 0.0f;
#pragma unroll
    for (int g = 0; g < 8; ++g) if (g * 8 < nsl) {
#pragma unroll
      for (int q = 0; q < 8; ++q) sv[g * 8 + q] = (logits + (size_t)min(g * 8 + q, nsl - 1) * sstride)[e];
    }
    float v = sv[0];
#pragma unroll
    for (int q = 1; q < 64; ++q) if (q < nsl) v += sv[q];
    if (isnan(v)) v = -INFINITY;      // nan_clean
    L.lv[e] = v;
  }
  ROUTE_TS(5);
  lds_barrier(); ROUTE_TS(6);
  route_select(n_exp, k, L);
  ROUTE_TS(7);
  lds_barrier();
}
// softmax over the chosen logits in ascending expert id (soft_top); called by the whole workgroup after route_topk
__device__ __forceinline__ void route_weights(int k, RouteLds& L) {
  const int e = threadIdx.x;
  float mx = -INFINITY, ex = 1.0f;
  if (e < k) { for (int i = 0; i < k; ++i) mx = fmaxf(mx, L.s_val[i]); ex = isfinite(mx) ? expf(L.s_val[e] - mx) : 1.0f; L.r_val[e] = ex; }
  lds_barrier();
  if (e < k) {
    float w;
    if (!isfinite(mx)) w = 1.0f / (float)k;
    else { float sum = 0.0f; for (int i = 0; i < k; ++i) sum += L.r_val[i]; w = ex / sum; }
    L.s_w[e] = w;
  }
}

// ---- routing + expert gate/up: h[entry][r] = silu(gate[r] . x) * (up[r] . x) -------------------------------------------
// grid (row tiles, entries), 16 waves; entry = ti*(k+1) + j, j < k: the j-th chosen expert of token ti (ascending id),
// j == k: the shared expert.  Tile 0 of entry (ti, 0) publishes the token's expert ids and weights, tile 0 of the shared
// entry publishes the shared-expert gate sigmoid(sh_gate_inp . x).
// The K range is cut into P parts of NW wave shares each; a dot product is the sum of its parts in order from the
// first, a part the sum of its wave shares in wave order -- whatever the launch shape, so a token's result does not
// depend on it.  gridDim.z == 1: the workgroup's wave w takes share w of every part (P accumulators) and stores
// silu(g) * u.  gridDim.z == nz > 1 (P == 1 in the template, nz parts): workgroup kz takes part kz only -- an entry's 64
// rows on nz compute units instead of one; at one token a launch of tiles x (k+1) workgroups leaves most of the chip
// idle -- and leaves the part's raw sums, gate at h[((entry*nz + kz)*2 + 0)*hstride + row], up at [... + 1]; the down
// launch adds the parts and forms silu(g) * u with the same operations.
// The window form (PRE, both parts in the workgroup) is held to 64 registers for the formats whose decode fits them
// (next to) without spilling, so that two workgroups share a compute unit: five tokens' 440 workgroups are then resident
// at once instead of taking a second turn on the 256 compute units.
// PRE: the token's experts were chosen by k_moe_route (windows of several tokens: hundreds of workgroups would each redo
// the selection otherwise); the workgroup reads its expert id and publishes nothing but the shared-expert gate.
// FIX: the A3B configuration's constants (512 experts, top 10, d = 2048 in 32 router slices, ff = 512) folded in at compile
// time (the launcher checks them) -- same arithmetic.
// ID (IQ3_S): the dot products in the integer form of digits.h -- 1.4 vector instructions a weight where byte -> float and
// multiply-add take 3; dgx holds the digits of the window's activations, token ti at dgx + ti * (d / 64) * DGX_STRIDE.
template <int FMT, int NW, int P, bool PRE, bool FIX = false, bool ID = false>
__global__ __launch_bounds__(NW * 64, (PRE && P == 2 && FMT >= 5 && FMT <= 7) ? 8 : 1) void k_moe_gu(MoeDev m, const float* __restrict__ logits, int32_t* __restrict__ sel_idx, float* __restrict__ sel_w, float* __restrict__ sg,
                                                   const float* __restrict__ x, float* __restrict__ h, int hstride, const uint2* __restrict__ g2, int nsl, int sstride, int tstride, const uint32_t* __restrict__ dgx,
                                                   uint32_t* __restrict__ dgh) {
  static_assert(!ID || FMT == FMT_IQ3_S, "the integer form is IQ3_S's");
  const uint2* lds2 = nullptr;          // no format needs a codebook in shared memory any more
  PYRE_TS_VARS PYRE_TS(0);
  args_now(m.n_exp, m.top_k, logits, nsl, sstride, tstride);          // what the selection needs; the rest would crowd the scalar registers the activations go through
  const int n_exp = FIX ? 512 : m.n_exp, top_k = FIX ? 10 : m.top_k, d = FIX ? 2048 : m.d, ff = FIX ? 512 : m.ff;
  if constexpr (FIX) nsl = 32;
  __shared__ float red[2][P][NW][64];
  __shared__ RouteLds rl;
  __shared__ uint8_t hsm[ID ? 3 : 1][64];
  const int entry = blockIdx.y, k1 = top_k + 1, ti = entry / k1, j = entry % k1;
  const bool shared = j == top_k;
  const int nrows = shared ? m.sf : ff;
  if ((int)blockIdx.x * 64 >= nrows) return;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const float* xs = x + (size_t)ti * d;
  int expert = 0;
  if (!shared) {
    if constexpr (PRE) expert = __builtin_amdgcn_readfirstlane(sel_idx[ti * top_k + j]);
    else { route_topk(logits + (size_t)ti * tstride, nsl, sstride, n_exp, top_k, rl ROUTE_TS_ARG); expert = __builtin_amdgcn_readfirstlane(rl.s_idx[j]); }
  } else if (blockIdx.x == 0) {
    float p = 0.0f;
    for (int ib = threadIdx.x; ib < d; ib += 4 * NW * 64) {          // four elements per pass, loads first (elements past d: weight zero)
      float a[4], b[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) { const int ic = min(ib + u * NW * 64, d - 1); a[u] = m.sh_gate_inp[ic]; b[u] = xs[ic]; }
#pragma unroll
      for (int u = 0; u < 4; ++u) if (ib + u * NW * 64 < d) p = fmaf(a[u], b[u], p);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) p += __shfl_xor(p, o);
    if (lane == 0) red[0][0][wave][0] = p;
    lds_barrier();
    if (threadIdx.x == 0) { float tot = 0.0f; for (int w = 0; w < NW; ++w) tot += red[0][0][w][0]; rl.s_w[0] = 1.0f / (1.0f + expf(-tot)); }
    lds_barrier();
  }
  PYRE_TS(1);
  const QMatDev& G = shared ? m.sh_gate : m.gate_e; const QMatDev& Up = shared ? m.sh_up : m.up_e;
  const int tile = (shared ? 0 : expert * (ff >> 6)) + blockIdx.x;
  const int nz = (FIX && !PRE) ? 2 : (FIX ? 1 : (int)gridDim.z), kz = blockIdx.z, np = P * nz;          // np parts in all (FIX: two workgroups a single token's entry, one a window's)
  const int GU = FIX ? 32 : G.U;          // 64-column units of a row (both matrices, routed or shared: d / 64)
  const int upw = (GU + NW * np - 1) / (NW * np);
  const uint32_t* dgs = ID ? dgx + (size_t)ti * GU * DGX_STRIDE : nullptr;
  // one unit of a matrix into an accumulator, in the f32 or the integer form
  auto mac = [&](const QMatDev& Q, const UnitRaw<FMT>& r, int ku, float (&a)[1]) {
    if constexpr (ID) unit_idot_iq3s(r, dgs + (size_t)ku * DGX_STRIDE, a[0]);
    else unit_fma<FMT, 1>(Q, r, ku, lds2, lane, xs + ku * 64, 0, a);
  };
  float ag[P][1], au[P][1];
#pragma unroll
  for (int p = 0; p < P; ++p) { ag[p][0] = 0.0f; au[p][0] = 0.0f; }
  if (P == 2 && upw == 1) {
    // one unit per part: both parts' units of both matrices are fetched before the first is consumed
    const int ka = min(2 * wave, GU - 1), kb = min(2 * wave + 1, GU - 1);
    UnitRaw<FMT> g0 = unit_load<FMT>(G, tile, ka, lane), u0 = unit_load<FMT>(Up, tile, ka, lane), g1 = unit_load<FMT>(G, tile, kb, lane), u1 = unit_load<FMT>(Up, tile, kb, lane);
    if (2 * wave < GU) { mac(G, g0, ka, ag[0]); mac(Up, u0, ka, au[0]); }
    if (2 * wave + 1 < GU) { mac(G, g1, kb, ag[P - 1]); mac(Up, u1, kb, au[P - 1]); }
  } else {
#pragma unroll
    for (int p = 0; p < P; ++p) {
      const int k0 = min(GU, (wave * np + kz * P + p) * upw), kend = min(GU, k0 + upw);          // wave w's shares of the np parts are adjacent
      // two units of both matrices are fetched before the first is consumed: a rolled loop would pay a memory round trip per unit
      for (int ku = k0; ku < kend; ku += 2) {
        const int kb = min(ku + 1, kend - 1);
        UnitRaw<FMT> g0 = unit_load<FMT>(G, tile, ku, lane), u0 = unit_load<FMT>(Up, tile, ku, lane), g1 = unit_load<FMT>(G, tile, kb, lane), u1 = unit_load<FMT>(Up, tile, kb, lane);
        mac(G, g0, ku, ag[p]); mac(Up, u0, ku, au[p]);
        if (ku + 1 < kend) { mac(G, g1, ku + 1, ag[p]); mac(Up, u1, ku + 1, au[p]); }
      }
    }
  }
#pragma unroll
  for (int p = 0; p < P; ++p) { red[0][p][wave][lane] = ag[p][0]; red[1][p][wave][lane] = au[p][0]; }
  PYRE_TS(2);
  lds_barrier(); PYRE_TS(3);
  if (threadIdx.x < 64) {
    float g = 0.0f, u = 0.0f;
#pragma unroll
    for (int p = 0; p < P; ++p) {
      float gp = red[0][p][0][lane], up = red[1][p][0][lane];
#pragma unroll
      for (int w = 1; w < NW; ++w) { gp += red[0][p][w][lane]; up += red[1][p][w][lane]; }
      if (p == 0) { g = gp; u = up; } else { g += gp; u += up; }
    }
    if (nz == 1) {
      float s = 1.0f / (1.0f + expf(-g));
      const float hv = (g * s) * u;      // silu(g) * u, silu(x) = x * sigm(x)
      h[(size_t)entry * hstride + blockIdx.x * 64 + lane] = hv;
      // the tile's 64 rows are one unit of the down product's columns: their digits for its integer form
      if constexpr (ID) { if (dgh) digits_eo_wave(hv, lane, hsm, dgh + ((size_t)entry * (hstride >> 6) + blockIdx.x) * DGX_STRIDE); }
    } else {
      float* hp = h + ((size_t)entry * nz + kz) * 2 * hstride + blockIdx.x * 64 + lane;
      hp[0] = g; hp[hstride] = u;
    }
  }
  // Publishing comes last: a global store ahead of the dot products would stop the compiler from keeping the
  // activations in scalar registers (it could no longer prove them unmodified).
  if (blockIdx.x == 0 && kz == 0) {
    if (shared) { if (threadIdx.x == 0) sg[ti] = rl.s_w[0]; }
    else if (!PRE && j == 0) {
      route_weights(top_k, rl);       // thread e < k writes and then reads its own s_w entry
      if ((int)threadIdx.x < top_k) { sel_idx[ti * top_k + threadIdx.x] = rl.s_idx[threadIdx.x]; sel_w[ti * top_k + threadIdx.x] = rl.s_w[threadIdx.x]; }
    }
  }
  PYRE_TS(4); PYRE_TS_FLUSH(moe_ts, 0);
}

// ---- routing alone (windows of several tokens): grid t, 1024 threads; ids ascending and softmax weights of token ti ------
template <bool FIX = false>
__global__ __launch_bounds__(1024) void k_moe_route(MoeDev m, const float* __restrict__ logits, int32_t* __restrict__ sel_idx, float* __restrict__ sel_w, int nsl, int sstride, int tstride) {
  __shared__ RouteLds rl;
  const int ti = blockIdx.x;
  const int n_exp = FIX ? 512 : m.n_exp, top_k = FIX ? 10 : m.top_k;          // FIX: the A3B configuration (and 32 router slices), checked by the launcher
  if constexpr (FIX) nsl = 32;
#ifdef PYRE_PHASE_TS
  unsigned long long ts_[8];
#endif
  route_topk(logits + (size_t)ti * tstride, nsl, sstride, n_exp, top_k, rl ROUTE_TS_ARG);
  route_weights(top_k, rl);
  if ((int)threadIdx.x < top_k) { sel_idx[ti * top_k + threadIdx.x] = rl.s_idx[threadIdx.x]; sel_w[ti * top_k + threadIdx.x] = rl.s_w[threadIdx.x]; }
}

// ---- expert down: partial[entry][r] = down[r] . h[entry] ---------------------------------------------------------------
// NZ > 1: h arrives as the gate / up sums of NZ K parts (k_moe_gu with gridDim.z = NZ); each wave forms the 64 values of
// a unit, silu(sum of gate parts) * (sum of up parts), in its own slice of shared memory while the unit's weights are
// on their way (a wave's shared-memory operations execute in order: no workgroup barrier).
// ID (IQ3_S): the integer form of digits.h on the digits of h -- left by k_moe_gu beside h (NZ == 1), or formed here by
// the wave that forms the unit's values (NZ > 1); the same digits either way, so a token's bits do not depend on the form.
template <int FMT, int NW, int NZ, bool FIX = false, bool ID = false>
__global__ __launch_bounds__(NW * 64) void k_moe_down(MoeDev m, const int32_t* __restrict__ sel_idx, const float* __restrict__ h, int hstride, float* __restrict__ partial,
                                                     const uint2* __restrict__ g2, const uint32_t* __restrict__ dgh) {
  static_assert(!ID || FMT == FMT_IQ3_S, "the integer form is IQ3_S's");
  const uint2* lds2 = nullptr;          // no format needs a codebook in shared memory any more
  PYRE_TS_VARS PYRE_TS(0);
  qmat_args_now(m.down_e); qmat_args_now(m.sh_down); args_now(m.d, m.top_k, sel_idx, h, hstride, partial);
  const int top_k = FIX ? 10 : m.top_k, d = FIX ? 2048 : m.d;          // FIX: the A3B configuration (top 10, d = 2048, routed and shared experts 512 wide), checked by the launcher
  __shared__ float red[NW][64];
  __shared__ float hx[(NZ > 1 && !ID) ? NW : 1][64];
  __shared__ __align__(16) uint32_t hdg[(NZ > 1 && ID) ? NW : 1][DGX_STRIDE];
  __shared__ uint8_t hsm[(NZ > 1 && ID) ? NW : 1][3][64];
  const int entry = blockIdx.y, k1 = top_k + 1, ti = entry / k1, j = entry % k1;
  const bool shared = j == top_k;
  const QMatDev& D = shared ? m.sh_down : m.down_e;
  const int tile = (shared ? 0 : sel_idx[ti * top_k + j] * (d >> 6)) + blockIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int DU = FIX ? 8 : D.U;
  const int upw = (DU + NW - 1) / NW, k0 = wave * upw, kend = min(DU, k0 + upw);
  float acc[1] = {0.0f};
  if constexpr (NZ == 1) {
    const float* xs = h + (size_t)entry * hstride;
    if constexpr (ID) {
      const uint32_t* dge = dgh + (size_t)entry * (hstride >> 6) * DGX_STRIDE;
      for (int ku = k0; ku < kend; ++ku) { UnitRaw<FMT> r = unit_load<FMT>(D, tile, ku, lane); unit_idot_iq3s(r, dge + (size_t)ku * DGX_STRIDE, acc[0]); }
    } else
    for (int ku = k0; ku < kend; ++ku) unit_dot<FMT, 1>(D, lds2, tile, ku, lane, xs + ku * 64, 0, acc);
  } else {
    const float* hp = h + (size_t)entry * NZ * 2 * hstride + lane;
    for (int ku = k0; ku < kend; ++ku) {
      UnitRaw<FMT> r = unit_load<FMT>(D, tile, ku, lane);
      float gp[NZ], up[NZ];
#pragma unroll
      for (int q = 0; q < NZ; ++q) { gp[q] = hp[(size_t)(2 * q) * hstride + ku * 64]; up[q] = hp[(size_t)(2 * q + 1) * hstride + ku * 64]; }
      float g = gp[0], u = up[0];
#pragma unroll
      for (int q = 1; q < NZ; ++q) { g += gp[q]; u += up[q]; }
      float s = 1.0f / (1.0f + expf(-g));
      __builtin_amdgcn_wave_barrier();
      if constexpr (ID) {
        digits_eo_wave((g * s) * u, lane, hsm[wave], hdg[wave]);
        __builtin_amdgcn_wave_barrier();
        unit_idot_iq3s(r, hdg[wave], acc[0]);
      } else {
        hx[wave][lane] = (g * s) * u;
        __builtin_amdgcn_wave_barrier();
        unit_fma<FMT, 1>(D, r, ku, lds2, lane, hx[wave], 0, acc);
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
  red[wave][lane] = acc[0];
  PYRE_TS(1);
  lds_barrier(); PYRE_TS(2);
  if (threadIdx.x < 64) {
    float s = red[0][lane];
#pragma unroll
    for (int w = 1; w < NW; ++w) s += red[w][lane];
    partial[(size_t)entry * d + blockIdx.x * 64 + lane] = s;
  }
  PYRE_TS(3); PYRE_TS_FLUSH(moe_ts, 8);
}

// y[ti][r]: the four group sums of moe_out_value, added in order (few experts only: top_k <= PYRE_MOE_KMAX; more experts
// take the plain sum shared * sg + (the experts' terms in ascending id, from zero))
__global__ void k_moe_sum(const float* __restrict__ partial, const float* __restrict__ sel_w, const float* __restrict__ sg, int d, int k, float* __restrict__ y) {
  int r = blockIdx.x * blockDim.x + threadIdx.x, ti = blockIdx.y; if (r >= d) return;
  if (k <= PYRE_MOE_KMAX) { const MoeOut mo{partial, sel_w, sg, d, k}; y[(size_t)ti * d + r] = moe_out_value(mo, ti, r); return; }
  const float* p = partial + (size_t)ti * (k + 1) * d;
  float o = 0.0f; for (int j = 0; j < k; ++j) o += sel_w[ti * k + j] * p[(size_t)j * d + r];
  float yv = p[(size_t)k * d + r] * sg[ti];
  y[(size_t)ti * d + r] = yv + o;
}

// ---- expert down of a window, summed by groups: parts[(q*t + ti)*d + r] = P_q of moe_out_value -------------------------------
// grid (d/64, t, PYRE_MOE_GROUPS), NW waves.  The workgroup computes the down rows of its group's (at most PYRE_MOE_GMAX)
// entries as k_moe_down does -- wave w the K share w of every entry, the shares added in wave order -- and folds them with
// the routing weights in the group's order: the consumer then reads four vectors a token instead of k + 1, and the value is
// bit for bit what moe_out_value forms from k_moe_down's unreduced terms.  A wave's weights of all entries and its slices
// of their activations (through its own shared memory: no workgroup barrier) are fetched before the first is used.
// GE: entries a group can hold in this instance (3 covers top_k <= 11, PYRE_MOE_GMAX the rest) -- the register budget follows it.
// ID (IQ3_S): the integer form on the digits k_moe_gu left beside h, as k_moe_down<.., ID>.
template <int FMT, int NW, int GE, bool FIX = false, bool ID = false>
__global__ __launch_bounds__(NW * 64, (GE <= 3 && FMT >= 5 && FMT <= 7) ? 6 : 1) void k_moe_down_groups(MoeDev m, const int32_t* __restrict__ sel_idx, const float* __restrict__ sel_w, const float* __restrict__ sg,
                                                            const float* __restrict__ h, int hstride, float* __restrict__ parts, const uint2* __restrict__ g2, const uint32_t* __restrict__ dgh) {
  static_assert(GE <= PYRE_MOE_GMAX, "a group holds at most PYRE_MOE_GMAX entries");
  static_assert(!ID || FMT == FMT_IQ3_S, "the integer form is IQ3_S's");
  const uint2* lds2 = nullptr;
  qmat_args_now(m.down_e); qmat_args_now(m.sh_down); args_now(m.d, m.top_k, sel_idx, h, hstride, parts);
  __shared__ float red[GE][NW][64];
  __shared__ float hx[ID ? 1 : NW][GE][64];
  __shared__ __align__(16) uint32_t hdg[ID ? NW : 1][GE][DGX_STRIDE];
  const int ti = blockIdx.y, q = blockIdx.z, k = FIX ? 10 : m.top_k, gsz = (k + 4) / 4, d = FIX ? 2048 : m.d;          // FIX: the A3B configuration (top 10, d = 2048, experts 512 wide), checked by the launcher
  const int j0 = min(k, q * gsz), nr = min(k, j0 + gsz) - j0;          // the group's routed entries j0 .. j0+nr-1
  const bool with_shared = q == PYRE_MOE_GROUPS - 1;
  const int ne = nr + (with_shared ? 1 : 0);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  // the routed and the shared matrices may differ in width: each has its own K shares (as in k_moe_down)
  const int Ur = FIX ? 8 : m.down_e.U, Us = FIX ? 8 : m.sh_down.U, upr = (Ur + NW - 1) / NW, ups = (Us + NW - 1) / NW;
  const int niter = max(nr > 0 ? upr : 0, with_shared ? ups : 0);
  int tile[GE]; const float* xs[GE]; const uint32_t* dge[GE];
#pragma unroll
  for (int e = 0; e < GE; ++e) {
    const bool shared = with_shared && e == nr; const int j = shared ? k : min(j0 + e, k - 1);
    tile[e] = (shared ? 0 : __builtin_amdgcn_readfirstlane(sel_idx[ti * k + j]) * (d >> 6)) + blockIdx.x;
    xs[e] = h + (size_t)(ti * (k + 1) + j) * hstride;
    dge[e] = ID ? dgh + (size_t)(ti * (k + 1) + j) * (hstride >> 6) * DGX_STRIDE : nullptr;
  }
  float acc[GE][1];
#pragma unroll
  for (int e = 0; e < GE; ++e) acc[e][0] = 0.0f;
  // the routing weights and the shared expert's gate are requested now, not behind the products
  float wv[GE];
#pragma unroll
  for (int e = 0; e < GE; ++e) wv[e] = e < nr ? sel_w[ti * k + j0 + e] : 0.0f;
  const float g = with_shared ? sg[ti] : 0.0f;
  for (int it = 0; it < niter; ++it) {
    UnitRaw<FMT> r[GE]; float hv[GE]; bool on[GE]; int ku[GE];
#pragma unroll
    for (int e = 0; e < GE; ++e) {
      const bool shared = with_shared && e == nr; const int up = shared ? ups : upr, U = shared ? Us : Ur;
      ku[e] = wave * up + it; on[e] = e < ne && it < up && ku[e] < U;
      if (on[e]) { const QMatDev& D = shared ? m.sh_down : m.down_e; r[e] = unit_load<FMT>(D, tile[e], ku[e], lane); if constexpr (!ID) hv[e] = xs[e][ku[e] * 64 + lane]; }
    }
    if constexpr (ID) {
      // the units' digits through the wave's own shared memory: one coalesced load an entry, all in flight with the weights
      // (as scalar loads they would come one entry after the other: three entries' digits do not fit the scalar registers)
      uint32_t dv[GE];
#pragma unroll
      for (int e = 0; e < GE; ++e) dv[e] = on[e] ? (dge[e] + (size_t)ku[e] * DGX_STRIDE)[lane] : 0u;
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int e = 0; e < GE; ++e) if (on[e]) hdg[wave][e][lane] = dv[e];
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int e = 0; e < GE; ++e) if (on[e]) unit_idot_iq3s(r[e], hdg[wave][e], acc[e][0]);
      __builtin_amdgcn_wave_barrier();
    } else {
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int e = 0; e < GE; ++e) if (on[e]) hx[wave][e][lane] = hv[e];
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int e = 0; e < GE; ++e) if (on[e]) { const QMatDev& D = (with_shared && e == nr) ? m.sh_down : m.down_e; unit_fma<FMT, 1>(D, r[e], ku[e], lds2, lane, hx[wave][e], 0, acc[e]); }
      __builtin_amdgcn_wave_barrier();
    }
  }
#pragma unroll
  for (int e = 0; e < GE; ++e) if (e < ne) red[e][wave][lane] = acc[e][0];
  lds_barrier();
  if (threadIdx.x < 64) {
    float o = 0.0f;
#pragma unroll
    for (int e = 0; e < GE; ++e) if (e < ne) {
      float pv = red[e][0][lane];
#pragma unroll
      for (int w = 1; w < NW; ++w) pv += red[e][w][lane];
      if (e < nr) o = fmaf(wv[e], pv, o); else o = fmaf(pv, g, o);          // the shared expert comes last
    }
    parts[((size_t)q * gridDim.y + ti) * d + blockIdx.x * 64 + lane] = o;
  }
}

// the digits of t tokens' activations as a launch of its own (callers whose producer kernel does not leave them): grid (d / 64, t), one wave
__global__ __launch_bounds__(64) void k_act_digits_eo(const float* __restrict__ x, int d, uint32_t* __restrict__ dgx) {
  __shared__ uint8_t sm[3][64];
  const int ku = blockIdx.x, ti = blockIdx.y, lane = threadIdx.x;
  digits_eo_wave(x[(size_t)ti * d + ku * 64 + lane], lane, sm, dgx + ((size_t)ti * (d >> 6) + ku) * DGX_STRIDE);
}

#define PYRE_MOE_GU_NZMAX 2
size_t pyre_moe_work_bytes(const MoeDev& m) {
  size_t hs = (size_t)(m.ff > m.sf ? m.ff : m.sf), k1 = m.top_k + 1;
  return 256 * 11 + sizeof(float) * (8 * (size_t)m.n_exp + 8 * (size_t)m.top_k * 2 + 8 + 8 * k1 * hs * 2 * PYRE_MOE_GU_NZMAX + 8 * k1 * (size_t)m.d + 8 * PYRE_MOE_GROUPS * (size_t)m.d + 8 * (size_t)(m.d / 64) * DGX_STRIDE + 8 * k1 * (hs / 64) * DGX_STRIDE);
}
void pyre_moe_work_carve(const MoeDev& m, void* base, MoeWork* w) {
  uint8_t* p = (uint8_t*)base; auto take = [&](size_t n) { void* r = p; p += (n + 255) & ~(size_t)255; return r; };
  size_t hs = (size_t)(m.ff > m.sf ? m.ff : m.sf), k1 = m.top_k + 1;
  w->logits = (float*)take(4 * 8 * (size_t)m.n_exp); w->sel_idx = (int32_t*)take(4 * 8 * (size_t)m.top_k); w->sel_w = (float*)take(4 * 8 * (size_t)m.top_k);
  w->sg = (float*)take(4 * 8); w->h = (float*)take(4 * 8 * k1 * hs * 2 * PYRE_MOE_GU_NZMAX); w->partial = (float*)take(4 * 8 * k1 * (size_t)m.d);
  w->parts = (float*)take(4 * 8 * PYRE_MOE_GROUPS * (size_t)m.d);
  w->dgx = (uint32_t*)take(4 * 8 * (size_t)(m.d / 64) * DGX_STRIDE);
  w->dgh = (uint32_t*)take(4 * 8 * k1 * (hs / 64) * DGX_STRIDE);
}

#define MOE_FMT_DISPATCH(fmt, CALL) \
  switch (fmt) { case FMT_F32: { constexpr int F = FMT_F32; CALL; } break; case FMT_F16: { constexpr int F = FMT_F16; CALL; } break; case FMT_BF16: { constexpr int F = FMT_BF16; CALL; } break; \
    case FMT_Q8_0: { constexpr int F = FMT_Q8_0; CALL; } break; case FMT_Q4_K: { constexpr int F = FMT_Q4_K; CALL; } break; case FMT_IQ2_XS: { constexpr int F = FMT_IQ2_XS; CALL; } break; \
    case FMT_C4: { constexpr int F = FMT_C4; CALL; } break; case FMT_C8: { constexpr int F = FMT_C8; CALL; } break; \
    default: { constexpr int F = FMT_IQ3_S; CALL; } break; }

// K parts of the gate/up dot products (a property of the matrices, so that every window length gives a token the
// same bits) and whether a window of t tokens launches one workgroup per part: only a single token does, whose
// tiles x (k+1) workgroups would leave most of the chip idle.
int pyre_moe_gu_parts(const MoeDev& m) {
  static const bool off = getenv("PYRE_MOE_GU_PARTS") && atoi(getenv("PYRE_MOE_GU_PARTS")) == 0;
  return (!off && m.gate_e.U % 32 == 0 && m.sh_gate.U == m.gate_e.U) ? 2 : 1;
}
int pyre_moe_launch(pyre_ctx* ctx, const MoeDev& m, const MoeWork& w, const float* x, int t, float* y, const RouteSrc* routed, bool in_groups) {
  if (in_groups && (y || t < 2 || !pyre_moe_groups_ok(m))) return pyre_fail(ctx, PYRE_E_ARG, "moe_ffn: group sums are for unreduced windows of 2..8 tokens with top_k <= %d", PYRE_MOE_KMAX);
  if (t < 1 || t > 8) return pyre_fail(ctx, PYRE_E_ARG, "moe_ffn: t = %d outside 1..8", t);
  if (!y && m.top_k > PYRE_MOE_KMAX) return pyre_fail(ctx, PYRE_E_SHAPE, "moe_ffn: an unreduced output needs top_k <= %d", PYRE_MOE_KMAX);
  if (routed && (routed->nsl < 1 || routed->nsl > 64 || routed->r64 < m.n_exp)) return pyre_fail(ctx, PYRE_E_ARG, "moe_ffn: %d router slices of %d rows", routed->nsl, routed->r64);
  if (t > 1 && getenv("PYRE_DEBUG_SKIP_MOE")) return PYRE_OK;
  if (!routed) { int rc = pyre_gemv_launch(ctx, m.router, x, t, w.logits); if (rc) return rc; }
  const float* lg = routed ? routed->p : w.logits; const int nsl = routed ? routed->nsl : 1, sstride = routed ? t * routed->r64 : 0, tstride = routed ? routed->r64 : m.n_exp;
  auto mat_bytes = [](const QMatDev& q, double rows) { return qmat_gguf_bytes(q, rows); };
  const int hs = m.ff > m.sf ? m.ff : m.sf, entries = t * (m.top_k + 1);
  const uint2* g2 = (const uint2*)ctx->d_iq2xs;
  const int P = pyre_moe_gu_parts(m), nz = (P > 1 && t == 1) ? P : 1;
  // IQ3_S experts: gate/up in the integer form, on the digits the mix left beside the activations or on a launch of their own
  static const bool idot_on = !(getenv("PYRE_MOE_IDOT") && atoi(getenv("PYRE_MOE_IDOT")) == 0);
  const bool idot = idot_on && m.gate_e.fmt == FMT_IQ3_S && m.sh_gate.fmt == FMT_IQ3_S;
  const uint32_t* dgx = nullptr;
  if (idot) {
    if (routed && routed->dgx) dgx = routed->dgx;
    else { ProfScope ps(ctx, "moe_digits", 4.0 * t * m.d * 2); hipLaunchKernelGGL(k_act_digits_eo, dim3(m.d / 64, t), dim3(64), 0, ctx->stream, x, m.d, w.dgx); PYRE_CHECK_LAUNCH(ctx); dgx = w.dgx; }
  }
  // ... and the down products on the digits of h, which a window's gate/up launch leaves and a single token's down launch forms
  static const bool idot_gu_only = getenv("PYRE_MOE_IDOT") && atoi(getenv("PYRE_MOE_IDOT")) == 1;
  const bool idot_dn = idot && !idot_gu_only && m.down_e.fmt == FMT_IQ3_S && m.sh_down.fmt == FMT_IQ3_S;
  uint32_t* dgh = idot_dn ? w.dgh : nullptr;
  const bool a3b = t == 1 && m.gate_e.fmt == FMT_IQ3_S && m.down_e.fmt == FMT_IQ3_S && m.n_exp == 512 && m.top_k == 10 && m.d == 2048 && m.ff == 512 && m.sf == 512;          // the instances with these constants folded in
  { ProfScope ps(ctx, "moe_route_gate_up", t * (2.0 * m.top_k * mat_bytes(m.gate_e, m.ff) + 2.0 * mat_bytes(m.sh_gate, m.sf)) + 4.0 * t * (m.n_exp + 2.0 * m.d));
#define GU_ARGS(NZ) dim3(hs / 64, entries, NZ), dim3(16 * 64), 0, ctx->stream, m, lg, w.sel_idx, w.sel_w, w.sg, x, w.h, hs, g2, nsl, sstride, tstride, dgx, dgh
#define GU_GO(PP, NZ, PRE) do { if (idot) hipLaunchKernelGGL((k_moe_gu<FMT_IQ3_S, 16, PP, PRE, false, true>), GU_ARGS(NZ)); else MOE_FMT_DISPATCH(m.gate_e.fmt, hipLaunchKernelGGL((k_moe_gu<F, 16, PP, PRE>), GU_ARGS(NZ))); } while (0)
  if (t == 1 && a3b && nsl == 32 && nz == 2) { if (idot) hipLaunchKernelGGL((k_moe_gu<FMT_IQ3_S, 16, 1, false, true, true>), GU_ARGS(2)); else hipLaunchKernelGGL((k_moe_gu<FMT_IQ3_S, 16, 1, false, true>), GU_ARGS(2)); }
  else if (t == 1) { GU_GO(1, nz, false); }          // the selection inside the launch; one workgroup per K part
  else {
    const bool a3bw = m.gate_e.fmt == FMT_IQ3_S && m.down_e.fmt == FMT_IQ3_S && m.n_exp == 512 && m.top_k == 10 && m.d == 2048 && m.ff == 512 && m.sf == 512 && nsl == 32;          // a window of the A3B configuration: constants folded in
    if (a3bw) hipLaunchKernelGGL(k_moe_route<true>, dim3(t), dim3(1024), 0, ctx->stream, m, lg, w.sel_idx, w.sel_w, nsl, sstride, tstride);
    else hipLaunchKernelGGL(k_moe_route<false>, dim3(t), dim3(1024), 0, ctx->stream, m, lg, w.sel_idx, w.sel_w, nsl, sstride, tstride);
    if (a3bw && P == 2) { if (idot) hipLaunchKernelGGL((k_moe_gu<FMT_IQ3_S, 16, 2, true, true, true>), GU_ARGS(1)); else hipLaunchKernelGGL((k_moe_gu<FMT_IQ3_S, 16, 2, true, true>), GU_ARGS(1)); }
    else if (P == 2) { GU_GO(2, 1, true); } else { GU_GO(1, 1, true); }
  } }
#undef GU_GO
#undef GU_ARGS
  PYRE_CHECK_LAUNCH(ctx);
  { ProfScope ps(ctx, "moe_down", t * (m.top_k * mat_bytes(m.down_e, m.d) + mat_bytes(m.sh_down, m.d)));
  if (in_groups) {
    const int gsz = (m.top_k + 4) / 4, last = m.top_k - min(m.top_k, (PYRE_MOE_GROUPS - 1) * gsz) + 1;          // entries of a full group, of the last (with the shared expert)
#define DOWN_G_GO(GE) MOE_FMT_DISPATCH(m.down_e.fmt, hipLaunchKernelGGL((k_moe_down_groups<F, 8, GE>), dim3(m.d / 64, t, PYRE_MOE_GROUPS), dim3(8 * 64), 0, ctx->stream, m, w.sel_idx, w.sel_w, w.sg, w.h, hs, w.parts, g2, dgh))
#define DOWN_G_ARGS dim3(m.d / 64, t, PYRE_MOE_GROUPS), dim3(8 * 64), 0, ctx->stream, m, w.sel_idx, w.sel_w, w.sg, w.h, hs, w.parts, g2, dgh
    if (m.gate_e.fmt == FMT_IQ3_S && m.down_e.fmt == FMT_IQ3_S && m.n_exp == 512 && m.top_k == 10 && m.d == 2048 && m.ff == 512 && m.sf == 512) {          // the A3B configuration: constants folded in
      if (idot_dn) hipLaunchKernelGGL((k_moe_down_groups<FMT_IQ3_S, 8, 3, true, true>), DOWN_G_ARGS); else hipLaunchKernelGGL((k_moe_down_groups<FMT_IQ3_S, 8, 3, true>), DOWN_G_ARGS);
    } else if (idot_dn) { if (gsz <= 3 && last <= 3) hipLaunchKernelGGL((k_moe_down_groups<FMT_IQ3_S, 8, 3, false, true>), DOWN_G_ARGS); else hipLaunchKernelGGL((k_moe_down_groups<FMT_IQ3_S, 8, PYRE_MOE_GMAX, false, true>), DOWN_G_ARGS); }
    else if (gsz <= 3 && last <= 3) { DOWN_G_GO(3); } else { DOWN_G_GO(PYRE_MOE_GMAX); }
#undef DOWN_G_ARGS
#undef DOWN_G_GO
  }
#define DOWN_ARGS dim3(m.d / 64, entries), dim3(8 * 64), 0, ctx->stream, m, w.sel_idx, w.h, hs, w.partial, g2, dgh
  else if (a3b && nz == 2) { if (idot_dn) hipLaunchKernelGGL((k_moe_down<FMT_IQ3_S, 8, 2, true, true>), DOWN_ARGS); else hipLaunchKernelGGL((k_moe_down<FMT_IQ3_S, 8, 2, true>), DOWN_ARGS); }
  else if (idot_dn) { if (nz == 1) hipLaunchKernelGGL((k_moe_down<FMT_IQ3_S, 8, 1, false, true>), DOWN_ARGS); else hipLaunchKernelGGL((k_moe_down<FMT_IQ3_S, 8, 2, false, true>), DOWN_ARGS); }
  else if (nz == 1) { MOE_FMT_DISPATCH(m.down_e.fmt, hipLaunchKernelGGL((k_moe_down<F, 8, 1>), DOWN_ARGS)); }
  else { MOE_FMT_DISPATCH(m.down_e.fmt, hipLaunchKernelGGL((k_moe_down<F, 8, 2>), DOWN_ARGS)); } }
#undef DOWN_ARGS
  PYRE_CHECK_LAUNCH(ctx);
  if (y) {
    ProfScope ps(ctx, "moe_sum", 4.0 * t * m.d * (m.top_k + 2));
    hipLaunchKernelGGL(k_moe_sum, dim3((m.d + 255) / 256, t), dim3(256), 0, ctx->stream, w.partial, w.sel_w, w.sg, m.d, m.top_k, y);
    PYRE_CHECK_LAUNCH(ctx);
  }
  return PYRE_OK;
}

// ---- the FFN of a block of prompt windows, the tokens grouped by expert ------------------------------------------------------
// A long prompt is run layer by layer over blocks of up to 32 windows of eight tokens (model.hip); between a layer's FFN mixes
// and the next layer the FFN of all of the block's tokens runs here: an expert's weights are fetched once for all of its
// tokens (a window by itself picks eight tokens x 10 of 512 experts and shares nothing).  A token's arithmetic is that of
// the window kernels above, in the same order (k_moe_route, k_moe_gu<.., 2, true, .., ID>, k_moe_down_groups<.., ID>): its
// bits do not depend on which path ran.  IQ3_S experts in the integer form only, gate / up rows of 32 units, expert widths
// of at most 8 units.
template <bool FIX>
__global__ __launch_bounds__(1024) void k_moe_route_blk(MoeDev m, MoeBlk b, int nsl, int r64) {
  __shared__ RouteLds rl;
  const int ti = blockIdx.x, w = ti >> 3, tw = ti & 7;
  const int n_exp = FIX ? 512 : m.n_exp, top_k = FIX ? 10 : m.top_k;
  if constexpr (FIX) nsl = 32;
#ifdef PYRE_PHASE_TS
  unsigned long long ts_[8];
#endif
  route_topk(b.rpart + (size_t)w * b.ws + (size_t)tw * r64, nsl, 8 * r64, n_exp, top_k, rl ROUTE_TS_ARG);
  route_weights(top_k, rl);
  if ((int)threadIdx.x < top_k) { b.sel_idx[ti * top_k + threadIdx.x] = rl.s_idx[threadIdx.x]; b.sel_w[ti * top_k + threadIdx.x] = rl.s_w[threadIdx.x]; }
}
// The router's K-slice sums of a block when they do not ride on the windows' FFN mixes: grid (d / 64, T / 8), 4 waves.  The
// workgroup stages its window's eight tokens' 64 columns of x and forms, tile of 64 experts by tile, the partial dot products
// the riding code of k_hc_up_mix_m forms (unit_fma over the same 64 values in the same order): the same bits, where the
// windows' path has them.
template <int RF>
__global__ __launch_bounds__(256) void k_moe_router_blk(MoeDev m, MoeBlk b, int r64) {
  __shared__ float xs[8][64];
  const uint2* lds2 = nullptr;
  const int sl = blockIdx.x, w = blockIdx.y, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const float* xw = b.x + (size_t)w * b.ws;
  for (int i = threadIdx.x; i < 8 * 64; i += 256) xs[i >> 6][i & 63] = xw[(size_t)(i >> 6) * m.d + sl * 64 + (i & 63)];
  lds_barrier();
  float* rp = const_cast<float*>(b.rpart) + (size_t)w * b.ws;
  for (int tile = wave; tile < m.router.tiles; tile += 4) {
    const UnitRaw<RF> rraw = unit_load<RF>(m.router, tile, sl, lane);
#pragma unroll 1
    for (int t2 = 0; t2 < 8; ++t2) {
      float ra[1] = {0.0f};
      unit_fma<RF, 1>(m.router, rraw, sl, lds2, lane, xs[t2], 0, ra);
      rp[((size_t)sl * 8 + t2) * r64 + (size_t)tile * 64 + lane] = ra[0];
    }
  }
}
// the (token, choice) pairs of the block by expert: eoff[e] .. eoff[e + 1] of elist hold expert e's entries token * (k + 1) + j
// (in no particular order: a token's sums do not depend on its neighbours).  One workgroup of 1024 threads.
__global__ __launch_bounds__(1024) void k_moe_lists(MoeDev m, MoeBlk b, int T) {
  __shared__ int cnt[1024], cur[1024];
  const int tid = threadIdx.x, k = m.top_k, np = T * k;
  cnt[tid] = 0;
  __syncthreads();
  for (int p = tid; p < np; p += 1024) atomicAdd(&cnt[b.sel_idx[p]], 1);
  __syncthreads();
  const int own = cnt[tid]; int v = own;
  for (int o = 1; o < 1024; o <<= 1) { cur[tid] = v; __syncthreads(); const int a = tid >= o ? cur[tid - o] : 0; __syncthreads(); v += a; }
  cur[tid] = v - own;            // exclusive prefix
  if (tid <= m.n_exp) b.eoff[tid] = tid < m.n_exp ? v - own : np;
  __syncthreads();
  for (int p = tid; p < np; p += 1024) { const int pos = atomicAdd(&cur[b.sel_idx[p]], 1); b.elist[pos] = (p / k) * (k + 1) + p % k; }
}
// What a workgroup of the two kernels below works on: blockIdx.y < n_exp: the routed expert's entries; above: eight tokens'
// entries of the shared expert.
struct BlkEntries { int n; const int32_t* list; int first; int step; };
__device__ __forceinline__ BlkEntries blk_entries(const MoeDev& m, const MoeBlk& b, int T, int ye) {
  BlkEntries e;
  if (ye < m.n_exp) { const int e0 = b.eoff[ye]; e.n = b.eoff[ye + 1] - e0; e.list = b.elist + e0; e.first = 0; e.step = 0; }
  else { const int t0 = (ye - m.n_exp) * 8; e.n = min(8, T - t0); e.list = nullptr; e.first = t0 * (m.top_k + 1) + m.top_k; e.step = m.top_k + 1; }
  return e;
}
__device__ __forceinline__ int blk_entry(const BlkEntries& e, int i) { return e.list ? e.list[i] : e.first + i * e.step; }

// f32 rows -> the matrix cores' operand, a row at a time: row r of x [n][cols] as its two f16 halves xh[r][0 / 1][cols], each
// 256-column stretch on its own power of two (the arithmetic of k_act_split, gemm_m.hip), the inverse factors in
// inv[r][cols / 256].  x2 given: the row is silu(x) * x2 (an expert's h out of its gate and up products).  gate_inp given:
// sg[r] = sigmoid(gate_inp . x[r]) as well (the shared expert's gate).  grid (n), 256 threads, a stretch a round.  Row n of
// xh is kept zero by the owner: the operand rows a pass has no token for point there.
__global__ __launch_bounds__(256) void k_blk_split(const float* __restrict__ x, const float* __restrict__ x2, int cols, uint16_t* __restrict__ xh, float* __restrict__ inv, const float* __restrict__ gate_inp, float* __restrict__ sg, size_t ws) {      // ws > 0: row r of x at x + (r / 8) * ws + (r % 8) * cols (a window's eight rows in its workspace)
  __shared__ float mx[2][4]; __shared__ float dp[4];
  const int r = blockIdx.x, i = threadIdx.x, wave = i >> 6, lane = i & 63;
  float dot = 0.0f;
  for (int sb = 0; sb < (cols >> 8); ++sb) {
    const int k = sb * 256 + i;
    float v = (ws ? x + (size_t)(r >> 3) * ws + (size_t)(r & 7) * cols : x + (size_t)r * cols)[k];
    if (x2) { const float sgm = 1.0f / (1.0f + expf(-v)); v = (v * sgm) * x2[(size_t)r * cols + k]; }
    if (gate_inp) dot = fmaf(gate_inp[k], v, dot);
    float a = fabsf(v); a = a == a ? a : INFINITY;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) a = fmaxf(a, __shfl_xor(a, o));
    if (lane == 0) mx[sb & 1][wave] = a;
    __syncthreads();            // (the two halves of mx take turns: one barrier a round)
    const float mv = fmaxf(fmaxf(mx[sb & 1][0], mx[sb & 1][1]), fmaxf(mx[sb & 1][2], mx[sb & 1][3]));
    int e = 0;
    if (mv > 0.0f && mv < INFINITY) { e = 140 - (int)((__float_as_uint(mv) >> 23) & 0xFF); e = e > 100 ? 100 : e; }
    const float up = __uint_as_float((uint32_t)(127 + e) << 23), dn = __uint_as_float((uint32_t)(127 - e) << 23);
    const float xs = v * up;
    const _Float16 h1 = (_Float16)xs, h2 = (_Float16)((xs - (float)h1) * 2048.0f);
    xh[((size_t)r * 2) * cols + k] = __builtin_bit_cast(unsigned short, h1); xh[((size_t)r * 2 + 1) * cols + k] = __builtin_bit_cast(unsigned short, h2);
    if (i == 0) inv[(size_t)r * (cols >> 8) + sb] = dn;
  }
  if (gate_inp) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) dot += __shfl_xor(dot, o);
    if (lane == 0) dp[wave] = dot;
    __syncthreads();
    if (i == 0) sg[r] = 1.0f / (1.0f + expf(-(((dp[0] + dp[1]) + dp[2]) + dp[3])));
  }
}
// the sixteen operand rows of a pass for chunk c: lane (kg, r) takes the eight columns 32 s + 8 kg .. of half r & 1 of the row
// its slot r >> 1 names; the scale factors of the two slots whose sums the lane holds
__device__ __forceinline__ void load_a_rows(const uint16_t* __restrict__ p, const float* __restrict__ i0, const float* __restrict__ i1, int c, ABuf& b) {
#pragma unroll
  for (int s = 0; s < 4; ++s) b.a[s] = *(const uint4*)(p + c * 128 + s * 32);
  b.ai0 = i0[c >> 1]; b.ai1 = i1[c >> 1];
}

// The expert products of a block on the matrix cores.  DOWN = false: gate and up (blockIdx.z), grid (ff / 256, n_exp +
// ceil(T / 8), 2), operand rows of x by token, out g / u [entry][ff]; DOWN = true: grid (d / 256, same, 1), operand rows of h
// by entry, out the unreduced terms partial[entry][d].  4 waves, each with 64 rows of its expert's matrix (FMT_IQ3_S_M) of
// its own: the wave walks all of the row tile's 128-column chunks with two register buffers taking turns and writes its sums
// itself -- no shared memory, no barrier.  The workgroup's entries go through in passes of eight (sixteen operand rows); a
// weight is decoded once a pass, whatever the pass holds.
template <bool DOWN>
__global__ __launch_bounds__(256, 3) void k_moe_mm_blk(MoeDev m, MoeBlk b, int T, int zrow) {            // zrow: the operand's zero row
  const int ye = blockIdx.y; const bool shared = ye >= m.n_exp;
  const BlkEntries E = blk_entries(m, b, T, ye);
  if (E.n <= 0) return;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, k1 = m.top_k + 1;
  const QMatDev& W = DOWN ? (shared ? m.sh_down_m : m.down_m) : (blockIdx.z ? (shared ? m.sh_up_m : m.up_m) : (shared ? m.sh_gate_m : m.gate_m));
  const int rows = DOWN ? m.d : m.ff, kc = DOWN ? m.ff : m.d;
  const int rt = blockIdx.x * 4 + wave;            // the wave's row tile inside the expert
  if (rt * 64 >= rows) return;
  const uint16_t* opnd = DOWN ? b.hh : b.xh; const float* inv = DOWN ? b.hinv : b.xinv;
  float* out = DOWN ? b.partial : (blockIdx.z ? b.u : b.g);
  const int tile = (shared ? 0 : ye * (rows >> 6)) + rt;
  const int K128 = kc >> 7, nsb = kc >> 8;
  const NibK nk = nib_consts();
  const int kg = lane >> 4, r = lane & 15, slot = r >> 1, half = r & 1, q = lane >> 4;
  for (int i0 = 0; i0 < E.n; i0 += 8) {
    const int np = min(8, E.n - i0);
    auto row_of = [&](int sl) { const int en = blk_entry(E, i0 + sl); return DOWN ? en : en / k1; };
    const size_t myrow = slot < np ? (size_t)row_of(slot) : (size_t)zrow;
    const uint16_t* ap = opnd + (myrow * 2 + half) * kc + kg * 8;
    const bool on0 = 2 * q < np, on1 = 2 * q + 1 < np;
    const float* ip0 = inv + (size_t)(on0 ? row_of(2 * q) : 0) * nsb;            // (a slot without a token reads some row's factors: its sums are never written)
    const float* ip1 = inv + (size_t)(on1 ? row_of(2 * q + 1) : 0) * nsb;
    v4f tot[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) tot[g] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    WBuf<4> w0, w1; ABuf a0, a1;
    load_a_rows(ap, ip0, ip1, 0, a0); load_w<4>(W, tile * 4, 0, lane, K128, w0);
    for (int c = 0; c < K128; c += 2) {
      if (c + 1 < K128) { load_a_rows(ap, ip0, ip1, c + 1, a1); load_w<4>(W, tile * 4, c + 1, lane, K128, w1); }
      __builtin_amdgcn_sched_barrier(0);
      chunk_mac<4>(w0, a0, c, nk, tot);
      __builtin_amdgcn_sched_barrier(0);
      if (c + 2 < K128) { load_a_rows(ap, ip0, ip1, c + 2, a0); load_w<4>(W, tile * 4, c + 2, lane, K128, w0); }
      __builtin_amdgcn_sched_barrier(0);
      if (c + 1 < K128) chunk_mac<4>(w1, a1, c + 1, nk, tot);
      __builtin_amdgcn_sched_barrier(0);
    }
    // lane (q, j) holds, for row group g, token slot 2q (halves h1, h2 * 2^11 in rows 0, 1 of its four) and slot 2q + 1
    float* o0 = on0 ? out + (size_t)blk_entry(E, i0 + 2 * q) * rows + rt * 64 + r : nullptr;
    float* o1 = on1 ? out + (size_t)blk_entry(E, i0 + 2 * q + 1) * rows + rt * 64 + r : nullptr;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if (o0) o0[g * 16] = tot[g][0] + tot[g][1] * (1.0f / 2048.0f);
      if (o1) o1[g * 16] = tot[g][2] + tot[g][3] * (1.0f / 2048.0f);
    }
  }
}
// the four group sums of every token (moe_out_value's groups, folded as k_moe_down_groups folds them) into the token's
// window: grid (d / 256, T), thread = row
__global__ __launch_bounds__(256) void k_moe_groups_blk(MoeDev m, MoeBlk b, int T) {
  const int r = blockIdx.x * 256 + threadIdx.x, ti = blockIdx.y, k = m.top_k, d = m.d, gsz = (k + 4) / 4;
  if (r >= d) return;
  const float* pt = b.partial + (size_t)ti * (k + 1) * d + r;
  float* out = b.parts + (size_t)(ti >> 3) * b.ws + (size_t)(ti & 7) * d + r;
#pragma unroll
  for (int q = 0; q < PYRE_MOE_GROUPS; ++q) {
    const int j0 = min(k, q * gsz), nr = min(k, j0 + gsz) - j0;
    float o = 0.0f;
    for (int e = 0; e < nr; ++e) o = fmaf(b.sel_w[ti * k + j0 + e], pt[(size_t)(j0 + e) * d], o);
    if (q == PYRE_MOE_GROUPS - 1) o = fmaf(pt[(size_t)k * d], b.sg[ti], o);            // the shared expert comes last
    out[(size_t)q * 8 * d] = o;
  }
}

static bool is_m(const QMatDev& q) { return q.fmt == FMT_IQ3_S_M && q.mq && q.mh; }
bool pyre_moe_block_ok(const MoeDev& m) {
  return is_m(m.gate_m) && is_m(m.up_m) && is_m(m.down_m) && is_m(m.sh_gate_m) && is_m(m.sh_up_m) && is_m(m.sh_down_m) && m.d % 256 == 0 && m.ff % 256 == 0 && m.sf == m.ff &&
         m.n_exp <= 1023 && pyre_moe_groups_ok(m);
}
size_t pyre_moe_block_bytes(const MoeDev& m, int T) {
  const size_t hs = (size_t)m.ff, k1 = m.top_k + 1, n = (size_t)T, ne = n * k1;
  return 256 * 12 + 4 * (2 * n * m.top_k + n + 1024 + n * m.top_k + 2 * ne * hs + ne * (size_t)m.d + ne * (hs / 256) + n * (m.d / 256)) + 2 * (2 * (n + 1) * m.d + 2 * (ne + 1) * hs);
}
void pyre_moe_block_carve(const MoeDev& m, int T, void* base, MoeBlk* b) {
  uint8_t* p = (uint8_t*)base; auto take = [&](size_t n) { void* r = p; p += (n + 255) & ~(size_t)255; return r; };
  const size_t hs = (size_t)m.ff, k1 = m.top_k + 1, n = (size_t)T, ne = n * k1;
  b->sel_idx = (int32_t*)take(4 * n * m.top_k); b->sel_w = (float*)take(4 * n * m.top_k); b->sg = (float*)take(4 * n); b->eoff = (int32_t*)take(4 * 1024); b->elist = (int32_t*)take(4 * n * m.top_k);
  b->g = (float*)take(4 * ne * hs); b->u = (float*)take(4 * ne * hs); b->partial = (float*)take(4 * ne * (size_t)m.d);
  b->xh = (uint16_t*)take(2 * 2 * (n + 1) * m.d); b->xinv = (float*)take(4 * n * (m.d / 256));
  b->hh = (uint16_t*)take(2 * 2 * (ne + 1) * hs); b->hinv = (float*)take(4 * ne * (hs / 256));
}
// the rows no token owns: row T of xh, row T * (top_k + 1) of hh (once, when the block's scratch is made: for the largest T)
int pyre_moe_block_zero_rows(pyre_ctx* ctx, const MoeDev& m, const MoeBlk& b, int T) {
  const size_t hs = (size_t)m.ff, ne = (size_t)T * (m.top_k + 1);
  PYRE_HIP(ctx, hipMemsetAsync(b.xh + (size_t)2 * T * m.d, 0, 2 * 2 * (size_t)m.d, ctx->stream));
  PYRE_HIP(ctx, hipMemsetAsync(b.hh + 2 * ne * hs, 0, 2 * 2 * hs, ctx->stream));
  return PYRE_OK;
}
// T = 8 * windows tokens (T_max: the T the scratch was carved and its zero rows were set for); the router's K-slice sums (nsl
// slices of r64 rows a token) come from the mixes
int pyre_moe_block_launch(pyre_ctx* ctx, const MoeDev& m, const MoeBlk& b, int T, int T_max, int nsl, int r64, bool router_here) {
  if (!pyre_moe_block_ok(m) || T < 8 || T % 8 || T > T_max || nsl < 1 || nsl > 64 || r64 < m.n_exp) return pyre_fail(ctx, PYRE_E_ARG, "moe block: unsupported shape (T = %d, %d router slices)", T, nsl);
  const int hs = m.ff, ny = m.n_exp + (T + 7) / 8, ne = T * (m.top_k + 1), ne_max = T_max * (m.top_k + 1);
  const bool fix = m.n_exp == 512 && m.top_k == 10 && nsl == 32;
  if (router_here) {          // the router's K-slice sums were not left by the mixes: form them now
    if (nsl != m.d / 64 || (m.router.fmt != FMT_BF16 && m.router.fmt != FMT_F32)) return pyre_fail(ctx, PYRE_E_ARG, "moe block: the router's sums by %d slices, router format %d", nsl, m.router.fmt);
    ProfScope ps(ctx, "moe_block_router", qmat_gguf_bytes(m.router, m.router.rows) + 4.0 * T * (m.d + (double)nsl * r64));
    if (m.router.fmt == FMT_BF16) hipLaunchKernelGGL(k_moe_router_blk<FMT_BF16>, dim3(nsl, T / 8), dim3(256), 0, ctx->stream, m, b, r64);
    else hipLaunchKernelGGL(k_moe_router_blk<FMT_F32>, dim3(nsl, T / 8), dim3(256), 0, ctx->stream, m, b, r64);
    PYRE_CHECK_LAUNCH(ctx);
  }
  { ProfScope ps(ctx, "moe_block_route", 4.0 * T * nsl * m.n_exp);
    if (fix) hipLaunchKernelGGL(k_moe_route_blk<true>, dim3(T), dim3(1024), 0, ctx->stream, m, b, nsl, r64); else hipLaunchKernelGGL(k_moe_route_blk<false>, dim3(T), dim3(1024), 0, ctx->stream, m, b, nsl, r64);
    hipLaunchKernelGGL(k_moe_lists, dim3(1), dim3(1024), 0, ctx->stream, m, b, T);
    hipLaunchKernelGGL(k_blk_split, dim3(T), dim3(256), 0, ctx->stream, b.x, (const float*)nullptr, m.d, b.xh, b.xinv, m.sh_gate_inp, b.sg, b.ws); } PYRE_CHECK_LAUNCH(ctx);
  { ProfScope ps(ctx, "moe_block_gate_up", 2.0 * m.n_exp * qmat_gguf_bytes(m.gate_e, m.ff) + 2.0 * qmat_gguf_bytes(m.sh_gate, m.sf));
    hipLaunchKernelGGL(k_moe_mm_blk<false>, dim3((hs + 255) / 256, ny, 2), dim3(256), 0, ctx->stream, m, b, T, T_max);
    hipLaunchKernelGGL(k_blk_split, dim3(ne), dim3(256), 0, ctx->stream, (const float*)b.g, (const float*)b.u, hs, b.hh, b.hinv, (const float*)nullptr, (float*)nullptr, (size_t)0); } PYRE_CHECK_LAUNCH(ctx);
  { ProfScope ps(ctx, "moe_block_down", (double)m.n_exp * qmat_gguf_bytes(m.down_e, m.d) + qmat_gguf_bytes(m.sh_down, m.d));
    hipLaunchKernelGGL(k_moe_mm_blk<true>, dim3((m.d + 255) / 256, ny, 1), dim3(256), 0, ctx->stream, m, b, T, ne_max);
    hipLaunchKernelGGL(k_moe_groups_blk, dim3((m.d + 255) / 256, T), dim3(256), 0, ctx->stream, m, b, T); } PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}

// ---- C ABI -------------------------------------------------------------------------------------------------------------
struct pyre_moe { pyre_ctx* ctx; MoeDev dv; MoeWork w; void* work; float* gate_inp; float* xy; };

extern "C" {

int pyre_moe_create(pyre_ctx* ctx, int top_k, const pyre_qmat* router, const pyre_qmat* gate_e, const pyre_qmat* up_e, const pyre_qmat* down_e,
                    const float* sh_gate_inp_host, const pyre_qmat* sh_gate, const pyre_qmat* sh_up, const pyre_qmat* sh_down, pyre_moe** out) {
  if (!ctx || !out || !router || !gate_e || !up_e || !down_e || !sh_gate_inp_host || !sh_gate || !sh_up || !sh_down) return pyre_fail(ctx, PYRE_E_ARG, "pyre_moe_create: null argument");
  *out = nullptr;
  size_t d = router->cols, E = router->rows; if (E == 0 || gate_e->rows % E) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_moe_create: gate_exps rows %zu not a multiple of %zu experts", gate_e->rows, E);
  size_t ff = gate_e->rows / E, sf = sh_gate->rows;
  if (gate_e->cols != d || up_e->cols != d || up_e->rows != E * ff || down_e->rows != E * d || down_e->cols != ff || sh_gate->cols != d || sh_up->cols != d || sh_up->rows != sf ||
      sh_down->rows != d || sh_down->cols != sf) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_moe_create: inconsistent expert tensor shapes");
  if (ff % 64 || sf % 64 || d % 64) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_moe_create: d, expert and shared widths must be multiples of 64");
  if (top_k < 1 || top_k > 32 || (size_t)top_k > E || E > 1024) return pyre_fail(ctx, PYRE_E_ARG, "pyre_moe_create: top_k %d / experts %zu unsupported", top_k, E);
  if (gate_e->dv.fmt != up_e->dv.fmt || sh_gate->dv.fmt != gate_e->dv.fmt || sh_up->dv.fmt != gate_e->dv.fmt || sh_down->dv.fmt != down_e->dv.fmt)
    return pyre_fail(ctx, PYRE_E_TYPE, "pyre_moe_create: gate/up (and shared gate/up) must share one type, down and shared down another");
  pyre_moe* m = new pyre_moe(); m->ctx = ctx;
  m->dv = MoeDev{router->dv, gate_e->dv, up_e->dv, down_e->dv, sh_gate->dv, sh_up->dv, sh_down->dv, nullptr, (int)d, (int)E, top_k, (int)ff, (int)sf};
  hipError_t e = hipMalloc((void**)&m->gate_inp, d * 4);
  if (e == hipSuccess) e = hipMemcpy(m->gate_inp, sh_gate_inp_host, d * 4, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMalloc(&m->work, pyre_moe_work_bytes(m->dv));
  if (e == hipSuccess) e = hipMalloc((void**)&m->xy, 2 * 8 * d * 4);
  if (e != hipSuccess) { int rc = pyre_fail(ctx, PYRE_E_HIP, "pyre_moe_create: %s", hipGetErrorString(e)); delete m; return rc; }
  m->dv.sh_gate_inp = m->gate_inp; pyre_moe_work_carve(m->dv, m->work, &m->w);
  *out = m; return PYRE_OK;
}
void pyre_moe_destroy(pyre_moe* m) { if (!m) return; (void)hipStreamSynchronize(m->ctx->stream); (void)hipFree(m->gate_inp); (void)hipFree(m->work); (void)hipFree(m->xy); delete m; }

int pyre_moe_ffn_dev(pyre_ctx* ctx, pyre_moe* m, const float* x_dev, int t, float* y_dev) {
  if (!ctx || !m || !x_dev || !y_dev) return pyre_fail(ctx, PYRE_E_ARG, "pyre_moe_ffn: null argument");
  return pyre_moe_launch(ctx, m->dv, m->w, x_dev, t, y_dev);
}
int pyre_moe_ffn(pyre_ctx* ctx, pyre_moe* m, const float* x_host, int t, float* y_host, int32_t* sel_idx_host, float* sel_w_host) {
  if (!ctx || !m || !x_host || !y_host) return pyre_fail(ctx, PYRE_E_ARG, "pyre_moe_ffn: null argument");
  if (t < 1 || t > 8) return pyre_fail(ctx, PYRE_E_ARG, "pyre_moe_ffn: t = %d outside 1..8", t);
  size_t n = (size_t)t * m->dv.d * 4; float* xd = m->xy; float* yd = m->xy + 8 * (size_t)m->dv.d;
  PYRE_HIP(ctx, hipMemcpyAsync(xd, x_host, n, hipMemcpyHostToDevice, ctx->stream));
  int rc = pyre_moe_launch(ctx, m->dv, m->w, xd, t, yd); if (rc) return rc;
  PYRE_HIP(ctx, hipMemcpyAsync(y_host, yd, n, hipMemcpyDeviceToHost, ctx->stream));
  if (sel_idx_host) PYRE_HIP(ctx, hipMemcpyAsync(sel_idx_host, m->w.sel_idx, (size_t)t * m->dv.top_k * 4, hipMemcpyDeviceToHost, ctx->stream));
  if (sel_w_host) PYRE_HIP(ctx, hipMemcpyAsync(sel_w_host, m->w.sel_w, (size_t)t * m->dv.top_k * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}

}  // extern "C"
