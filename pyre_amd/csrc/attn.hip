// Gated full attention at decode: q/k RMSNorm + partial RoPE + KV append, softmax(q K^T / sqrt(hd)) V * sigmoid(gate)
// over a cache whose old positions are 4-bit (absmax per 32, kv4) and whose recent window is f32.
// Follows attn_core (dense branch), src/model/qwen4exp_gguf.rs:1558-1615, rope :1436-1439 / :529-533,
// kv4::pack / get, src/model/kv4.rs:12-42, and the packed/recent split of kv_push, qwen4exp_gguf.rs:1519-1520.
#include "formats.h"

__device__ __forceinline__ float a_sigm(float x) { return 1.0f / (1.0f + expf(-x)); }
PYRE_TS_DECL(attn_ts) PYRE_TS_EXPORT(attn_ts, pyre_debug_ts_attn)
#ifdef PYRE_PHASE_TS
// diagnostics build: start, end and hardware id of every workgroup of the last k_attn_decode launch
__device__ unsigned long long attn_wg[4096 * 10];
extern "C" int pyre_debug_attn_wg(unsigned long long* out) { return hipMemcpyFromSymbol(out, HIP_SYMBOL(attn_wg), sizeof(unsigned long long) * 4096 * 10) == hipSuccess ? 0 : -1; }
#endif

size_t pyre_packed_boundary(size_t n, int kv_bits, int recent) { if (kv_bits != 4 || n <= (size_t)recent + 64) return 0; return ((n - recent) / 64) * 64; }

// The positions that fall below the packed boundary when the context grows from pos to pos + 1 positions.
__device__ __forceinline__ bool kv_pack_step_range(const AttnDev& a, int pos, int* p0, int* p1) {
  const int n = pos + 1;
  *p1 = (a.kv_bits == 4 && n > a.kv_recent + 64) ? ((n - a.kv_recent) / 64) * 64 : 0;
  *p0 = (a.kv_bits == 4 && n - 1 > a.kv_recent + 64) ? ((n - 1 - a.kv_recent) / 64) * 64 : 0;
  return *p1 > *p0;
}
// kv4::pack (src/model/kv4.rs:12-42), thread gid of [p0, p1): one thread per (position, 32-value block, K or V)
template <int HD> __device__ __forceinline__ void kv_pack_thread(const AttnDev& a, const KvDev& kv, int p0, int p1, size_t gid) {
  const int bpr = a.nkv * HD / 32;                 // blocks per cache row
  size_t per = (size_t)(p1 - p0) * bpr;
  if (gid >= 2 * per) return;
  const bool is_v = gid >= per; if (is_v) gid -= per;
  const int pos = p0 + (int)(gid / bpr), blk = (int)(gid % bpr), kvh = blk / (HD / 32), bb = blk % (HD / 32);
  float x[32];
  for (int i = 0; i < 32; ++i) x[i] = is_v ? kv.vf[(size_t)pos * a.nkv * HD + (size_t)blk * 32 + i] : kv.kf[kv_blk((size_t)kvh * HD + bb * 32 + i, (size_t)a.nkv * HD, pos)];
  float m = 0.0f; for (int i = 0; i < 32; ++i) m = fmaxf(m, fabsf(x[i]));
  const float s = (m > 0.0f && isfinite(m)) ? m / 7.0f : 0.0f;
  for (int w = 0; w < 4; ++w) {
    uint32_t u = 0;
    for (int j = 0; j < 8; ++j) { int q = s > 0.0f ? (int)fminf(fmaxf(roundf(x[8 * w + j] / s), -7.0f), 7.0f) : 0; u |= ((uint32_t)q & 0xFu) << (4 * j); }
    if (is_v) kv.vq[(size_t)pos * (a.nkv * HD / 8) + (size_t)blk * 4 + w] = u;
    else kv.kq[kv_blk((size_t)kvh * (HD / 8) + bb * 4 + w, (size_t)a.nkv * (HD / 8), pos)] = u;
  }
  if (is_v) kv.vs[(size_t)pos * bpr + blk] = s; else kv.ks[kv_blk((size_t)kvh * (HD / 32) + bb, (size_t)a.nkv * (HD / 32), pos)] = s;
}

// grid (nkv + nh, t), hd threads.  Blocks 0..nkv-1: key head -> rms_inplace(kn) -> rope -> cache (and the raw value row);
// blocks nkv..: query head h -> rms_inplace(qn) -> rope -> q scratch.
// Blocks past nkv + nh (single-token steps at a device-side position): the 64-position packing step that the growth
// of the context by this token may make due (k_kv_pack's work, old positions only: it touches nothing the other
// blocks write), so a replayed step does not spend a launch on a check that almost always finds nothing to do.
// A query head also leaves as two f16 halves, q * 2^e = h1 + h2 (e: the head's largest magnitude lands in
// [2^13, 2^14); elements below 2^-3 after scaling keep fewer than 22 bits, 2^-27 of the largest), with 2^-e in qsc: the operand of the packed-key product.  Within
// each group of eight dims the halves are stored in the order 0 4 1 5 2 6 3 7, the order in which a 32-bit word of
// eight 4-bit keys unpacks into f16 pairs.
template <int HD>
__global__ __launch_bounds__(HD) void k_attn_prep(AttnDev a, KvDev kv, const float* __restrict__ qkv, int stride, int start, const int* __restrict__ posp, float* __restrict__ qout, uint16_t* __restrict__ qh, float* __restrict__ qsc, size_t wz_qkv, size_t wz_q) {
  __shared__ float buf[HD]; __shared__ float red[HD / 64]; __shared__ float redm[HD / 64];
  if (posp) start = *posp;
  if (gridDim.z > 1) {          // consecutive windows in one launch (a long prompt's blocks): window z's projection wz_qkv bytes, its query buffers wz_q bytes further on per window, its positions behind the window before
    const size_t z = blockIdx.z; start += (int)z * (int)gridDim.y;
    qkv = (const float*)((const char*)qkv + z * wz_qkv); qout = (float*)((char*)qout + z * wz_q); qh = (uint16_t*)((char*)qh + z * wz_q); qsc = (float*)((char*)qsc + z * wz_q);
  }
  const int b = blockIdx.x, ti = blockIdx.y, tid = threadIdx.x, pos = start + ti;
  if (b >= a.nkv + a.nh) {
    int p0, p1;
    if (ti == 0 && kv_pack_step_range(a, start, &p0, &p1)) kv_pack_thread<HD>(a, kv, p0, p1, (size_t)(b - a.nkv - a.nh) * HD + tid);
    return;
  }
  const bool is_k = b < a.nkv; const int h = is_k ? b : b - a.nkv;
  const float* row = qkv + (size_t)ti * stride;
  const float* src = is_k ? row + (size_t)a.nh * 2 * HD + (size_t)h * HD : row + (size_t)h * 2 * HD;
  float v = src[tid];
  // the norm weight, the rotation frequency and the value element are fetched now, ahead of the barriers
  const int half = a.n_rot / 2, ri = tid < half ? tid : tid - half;
  const float nwt = is_k ? a.kn[tid] : a.qn[tid], rinv = tid < a.n_rot ? a.rope_inv[ri] : 0.0f;
  const float vrow = is_k ? row[(size_t)a.nh * 2 * HD + (size_t)a.nkv * HD + (size_t)h * HD + tid] : 0.0f;
  float ss = wave_sum(v * v);
  if ((tid & 63) == 0) red[tid >> 6] = ss;
  __syncthreads();
  float tot = 0.0f;
#pragma unroll
  for (int i = 0; i < HD / 64; ++i) tot += red[i];
  const float sc = 1.0f / sqrtf(tot / (float)HD + a.eps);
  v = v * (sc * nwt);            // rms_inplace: x *= s * w
  buf[tid] = v;
  __syncthreads();
  if (tid < a.n_rot) {
    int i = ri;
    float ang = (float)pos * rinv;
    float sn = sinf(ang), cs = cosf(ang);
    if (a.mscale != 1.0f) { cs = cs * a.mscale; sn = sn * a.mscale; }      // YaRN magnitude factor, rope_cs (:529-533)
    float x0 = buf[i], x1 = buf[i + half];
    v = tid < half ? x0 * cs - x1 * sn : x1 * cs + x0 * sn;
  }
  if (is_k) {
    kv.kf[kv_blk((size_t)h * HD + tid, (size_t)a.nkv * HD, pos)] = v;
    kv.vf[(size_t)pos * a.nkv * HD + (size_t)h * HD + tid] = vrow;
  } else {
    qout[((size_t)ti * a.nh + h) * HD + tid] = v;
    float am = fabsf(v); am = am == am ? am : INFINITY;
    am = wave_max(am);
    if ((tid & 63) == 0) redm[tid >> 6] = am;
    __syncthreads();
    float m = redm[0];
#pragma unroll
    for (int i = 1; i < HD / 64; ++i) m = fmaxf(m, redm[i]);
    int e = 0;
    if (m > 0.0f && m < INFINITY) { e = 140 - (int)((__float_as_uint(m) >> 23) & 0xFF); e = e > 100 ? 100 : e; }
    const float xs = v * __uint_as_float((uint32_t)(127 + e) << 23);
    const _Float16 h1 = (_Float16)xs, h2 = (_Float16)(xs - (float)h1);
    uint16_t* o = qh + ((size_t)ti * a.nh + h) * 2 * HD + (tid & ~7) + ((tid & 3) * 2 + ((tid >> 2) & 1));
    o[0] = __builtin_bit_cast(unsigned short, h1); o[HD] = __builtin_bit_cast(unsigned short, h2);
    if (tid == 0) qsc[(size_t)ti * a.nh + h] = __uint_as_float((uint32_t)(127 - e) << 23);
  }
}

// kv4::pack for positions [p0, p1): one thread per (position, 32-value block, K or V).
// With posp the range is decided on the device: the positions that fall below the packed boundary when the context
// grows from *posp to *posp + 1 positions (nothing on most steps).
template <int HD>
__global__ void k_kv_pack(AttnDev a, KvDev kv, int p0, int p1, const int* __restrict__ posp) {
  if (posp && !kv_pack_step_range(a, *posp, &p0, &p1)) return;
  kv_pack_thread<HD>(a, kv, p0, p1, (size_t)blockIdx.x * blockDim.x + threadIdx.x);
}

__device__ __forceinline__ float nib_val(uint32_t w, int i) { return (float)(((int)(w << (28 - 4 * i))) >> 28); }   // sign-extended nibble i

// grid (chunks of 64*NPW positions, nkv, t), 256*NPW threads.  One workgroup serves the G query heads that share a KV
// head.  Wave (pw, dq) owns the 64 positions pw*64.. of the chunk and the 64 head dims dq*64.., so every cache element is read
// once per workgroup and each wave has all of its loads in flight at once (at decode sizes the step is bound by memory
// latency, not bandwidth).  Both products run on the fp32 matrix cores as 16x16x4 tiles with the G heads as the
// (zero-padded) 16 columns: the query and the softmax weights are then ordinary per-lane operands instead of
// wave-uniform values that would have to come through scalar loads or shared-memory broadcasts.
//   v_mfma_f32_16x16x4f32: lane l supplies A[i = l%16][k = l/16] and B[k = l/16][j = l%16], and holds
//   D[i = 4*(l/16) + r][j = l%16] in register r.
//  phase 1: D[position][head] += K[position][dim] q[head][dim]; step s of lane group kg stands for dim 16*kg + s, so a
//           lane's 16 dims are 4 float4 of q and 2 words of 4-bit keys.  The four dim quarters are added in order.
//  phase 2: chunk-local max / exp / sum per head (thread = position x head group)
//  phase 3: D[dim][head] += V[position][dim] e[position][head]; row i of tile dt stands for dim 4*i + dt, so a lane's
//           4 tiles are one float4 (or 4 nibbles of one word) per position.  The four position quarters are added in order.
// A window's tokens share the pass over the cache: the 16 columns hold the G heads of up to 16 / G tokens (token k of the
// pass in columns k*G .. k*G+G-1), each with its own view (token k sees one position more than token k-1) -- a column's
// sums do not depend on its neighbours, so a token's result is what a pass of its own gives.  The 4-bit boundary is a
// property of a token's view; when it moves inside a window (one window in 64 / t) the launch gives every token a pass
// of its own (tp = 1).
typedef float f4v __attribute__((ext_vector_type(4)));
typedef _Float16 h8v __attribute__((ext_vector_type(8)));
typedef _Float16 h2v __attribute__((ext_vector_type(2)));
// lane 2 * q + O of the caller's row of sixteen lanes, for every lane of the row (q = 0..3 unrolled by the caller)
template <int O> __device__ __forceinline__ int row_bcast(int v, int q) {
  switch (q) { case 0: return __builtin_amdgcn_update_dpp(0, v, 0x150 + O, 0xf, 0xf, true); case 1: return __builtin_amdgcn_update_dpp(0, v, 0x150 + O + 2, 0xf, 0xf, true);
    case 2: return __builtin_amdgcn_update_dpp(0, v, 0x150 + O + 4, 0xf, 0xf, true); default: return __builtin_amdgcn_update_dpp(0, v, 0x150 + O + 6, 0xf, 0xf, true); }
}
// eight 4-bit two's-complement fields of w -> eight f16 numbers in the order 0 4 1 5 2 6 3 7: field ^ 8 is the value + 8,
// or-ed into the mantissa of 1024 it is the f16 number 1032 + value, and one packed subtraction leaves the value
__device__ __forceinline__ h8v nib8_f16(uint32_t w) {
  const uint32_t x = w ^ 0x88888888u;
  const h2v off = {(_Float16)1032.0f, (_Float16)1032.0f};
  struct U4 { uint32_t v[4]; } u;
#pragma unroll
  for (int q = 0; q < 4; ++q) u.v[q] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2v, ((x >> (4 * q)) & 0x000F000Fu) | 0x64006400u) - off);
  return __builtin_bit_cast(h8v, u);
}
// NC: columns the buffers hold -- G for launches of one token a pass (tp = 1), 16 otherwise.
template <int HD, int G, int NC>
__global__ __launch_bounds__(256 * PYRE_ATTN_NPW, 4) void k_attn_decode(AttnDev a, KvDev kv, const float* __restrict__ qbuf, const uint16_t* __restrict__ qh, const float* __restrict__ qsc, int start, const int* __restrict__ posp, float* __restrict__ part_o, float* __restrict__ part_ml, int max_chunks, int t, int tp) {
  static_assert(HD == 256, "the wave layout assumes 4 x 64 head dims");
  constexpr int NPW = PYRE_ATTN_NPW, CH = PYRE_ATTN_CHUNK, NT = 256 * NPW;
  static_assert(4 * CH == NPW * HD, "the score and value partials share one buffer");
  __shared__ float red[4 * CH * NC];          // phase 1: [dq][position][column];  phase 3: [pw][column][dim]
  __shared__ __align__(16) float sc[NC][CH + 4];          // [column][position]: eight consecutive positions of a column are two 16-byte reads
  __shared__ float wmax[NPW][NC], wsum[NPW][NC];
  PYRE_TS_VARS PYRE_TS(0);
  // Workgroups in dispatch order (x fastest): chunks descending, the KV heads of a chunk next to each other.  The
  // workgroups past the view (a captured launch covers the whole cache) leave first; the chunks of the f32 window, which
  // move eight times the bytes of a packed chunk, follow as neighbours in the order and so land on different compute
  // units, where each later shares its unit with a packed chunk instead of another f32 one.
  const int lin = (int)blockIdx.x + (int)gridDim.x * (int)blockIdx.y;
  const int chunk = (int)gridDim.x - 1 - lin / (int)gridDim.y, kvh = lin % (int)gridDim.y, tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), pw = wave % NPW, dq = wave / NPW;
  if (posp) start = *posp;
  const int tk0 = blockIdx.z * tp, nk = min(tp, t - tk0), ncol = nk * G;          // tokens tk0 .. tk0+nk-1 in columns 0 .. ncol-1
  const int n = start + tk0 + nk;                                                  // the widest view of the pass
  if (chunk * CH >= n) return;
  const float scale = 1.0f / sqrtf((float)HD);
  const int li = lane & 15, lg = lane >> 4;
  const int row = a.nkv * HD;
  const int pb = (int)((a.kv_bits == 4 && n > a.kv_recent + 64) ? ((n - a.kv_recent) / 64) * 64 : 0);
  const int wbase = chunk * CH + pw * 64, p = wbase + lane;
  const bool packed = wbase < pb, active = wbase < n;
  const int ctok = li / G, chead = li - ctok * G;                                              // the lane's column: token of the pass, head of the group
  // The packed values do not depend on the scores: their loads go out with the keys', one memory round trip for both.
  // Lane (li, lg) of the value product stands for two dims of a scale block (word li & 3, nibbles 2 * (li >> 2) + m) at
  // the eight positions 8 * lg .. of a 32-position group: vw[g][b][p] is the word of position 32 * g + 8 * lg + p in block
  // dq * 2 + b.  vsl[g]: the scale of position 32 * g + 8 * lg + (li & 7) in block dq * 2 + (li >> 3); the lanes of a row of
  // sixteen hold the 8 x 2 scales the row needs and pass them round with row broadcasts.
  // All of it through buffer descriptors: one 32-bit offset per array and lane, the rest of an address is a constant
  // of the instruction or a scalar.
  const int pos = pw * 64 + lane;
  constexpr int GH = (NC + 3) / 4;
  // chunk-local max / exp / sum per head; called by every wave after the barrier that follows its scores
  auto softmax_phase = [&]() {
    float sv[GH];
#pragma unroll
    for (int gi = 0; gi < GH; ++gi) {
      const int c = dq + 4 * gi; sv[gi] = -INFINITY;
      if (c < ncol) {
        const bool valid = p < start + tk0 + c / G + 1;          // the column's token sees positions below its own + 1
        float v = ((red[((size_t)0 * CH + pos) * NC + c] + red[((size_t)1 * CH + pos) * NC + c]) + red[((size_t)2 * CH + pos) * NC + c]) + red[((size_t)3 * CH + pos) * NC + c];
        sv[gi] = valid ? v * scale : -INFINITY;
        const float m = wave_max(sv[gi]);
        if (lane == 0) wmax[pw][c] = m;
      }
    }
    __syncthreads();
#pragma unroll
    for (int gi = 0; gi < GH; ++gi) {
      const int c = dq + 4 * gi;
      if (c < ncol) {
        const bool valid = p < start + tk0 + c / G + 1;
        float mm = wmax[0][c];          // the chunk's maximum of the column: every thread takes it from the waves' maxima itself
#pragma unroll
        for (int q = 1; q < NPW; ++q) mm = fmaxf(mm, wmax[q][c]);
        float e = valid ? expf(sv[gi] - mm) : 0.0f; sc[c][pos] = e;
        const float l = wave_sum(e);
        if (lane == 0) wsum[pw][c] = l;
      }
    }
    __syncthreads();          // weights of every position visible; the score partials in `red` are dead
  };
  // A wave is on one of two paths for the whole kernel -- packed positions or f32 ones (the branch is scalar: wbase is a
  // wave's) -- each with its own registers; both pass the same four barriers.
  if (active && packed) {             // packed positions lie below the boundary, hence inside the view
    // Lane (li, lg) of the value product stands for two dims of a scale block (word li & 3, nibbles 2 * (li >> 2) + m) at
    // the eight positions 8 * lg .. of a 32-position group: vw[g][b][p] is the word of position 32 * g + 8 * lg + p in
    // block dq * 2 + b.  vsl[g]: the scale of position 32 * g + 8 * lg + (li & 7) in block dq * 2 + (li >> 3); the lanes of a
    // row of sixteen hold the 8 x 2 scales the row needs and pass them round with row broadcasts.  The values do not
    // depend on the scores: their loads go out with the keys', one memory round trip for both.  All of it through
    // buffer descriptors: one 32-bit offset per array and lane, the rest of an address is a constant or a scalar.
    uint32_t vw[2][2][8]; float vsl[2]; uint32_t kw[4][2]; float ksc[4][2];
    {
      // the descriptors start at the wave's 64 positions: every offset below is small
      const int vrow = (row / 8) * 4, srow = (row / 32) * 4;          // bytes of a position's packed values and of its scales
      const __amdgpu_buffer_rsrc_t rvq = __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)kv.vq + (size_t)wbase * vrow), 0, 0xFFFFFFFF, 0x00020000), rvs = __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)kv.vs + (size_t)wbase * srow), 0, 0xFFFFFFFF, 0x00020000);
      const __amdgpu_buffer_rsrc_t rkq = __builtin_amdgcn_make_buffer_rsrc((void*)(kv.kq + (size_t)(wbase >> 6) * (a.nkv * (HD / 8)) * 64), 0, 0xFFFFFFFF, 0x00020000), rks = __builtin_amdgcn_make_buffer_rsrc((void*)(kv.ks + (size_t)(wbase >> 6) * (a.nkv * (HD / 32)) * 64), 0, 0xFFFFFFFF, 0x00020000);
      const int vq_off = 8 * lg * vrow + (kvh * (HD / 8) + dq * 8 + (li & 3)) * 4, vs_off = (8 * lg + (li & 7)) * srow + (kvh * (HD / 32) + dq * 2 + (li >> 3)) * 4;
      const int kq_off = ((kvh * (HD / 8) + dq * 8 + lg) * 64 + li) * 4, ks_off = ((kvh * (HD / 32) + dq * 2) * 64 + li) * 4;
#pragma unroll
      for (int pt = 0; pt < 4; ++pt)
#pragma unroll
        for (int b = 0; b < 2; ++b) {          // key word (block dq*2 + b, dims 8*lg ..) and block scale of position wbase + 16*pt + li
          kw[pt][b] = __builtin_amdgcn_raw_buffer_load_b32(rkq, kq_off, (b * 4 * 64 + 16 * pt) * 4, 0);
          ksc[pt][b] = __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(rks, ks_off, (b * 64 + 16 * pt) * 4, 0));
        }
#pragma unroll
      for (int g = 0; g < 2; ++g) {
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int q = 0; q < 8; ++q) vw[g][b][q] = __builtin_amdgcn_raw_buffer_load_b32(rvq, vq_off, (32 * g + q) * vrow + b * 16, 0);
        vsl[g] = __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(rvs, vs_off, 32 * g * srow, 0));
      }
    }
    PYRE_TS(1);
    {
      f4v D[4];
#pragma unroll
      for (int pt = 0; pt < 4; ++pt) D[pt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
      // 4-bit keys on the f16 matrix cores: one v_mfma_f32_16x16x32_f16 per query half covers 16 positions x a 32-dim
      // scale block.  A = the query halves (row = column of the pass), B = the keys (column = position, a lane's word
      // is its eight dims), so a lane's sums belong to its own position and meet that position's block scale in f32.
      // Products (4 bits x 11 bits) and the 32-term sums are exact in f32.
      h8v qa[2][2];
      if (li < ncol) {
        const uint4* qp = (const uint4*)(qh + ((size_t)(tk0 + ctok) * a.nh + (size_t)kvh * G + chead) * 2 * HD);
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int hf = 0; hf < 2; ++hf) qa[b][hf] = __builtin_bit_cast(h8v, qp[(hf * HD + (dq * 2 + b) * 32 + lg * 8) >> 3]);
      } else {
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int hf = 0; hf < 2; ++hf) qa[b][hf] = __builtin_bit_cast(h8v, make_uint4(0, 0, 0, 0));
      }
      float qinv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) { const int c = 4 * lg + r; qinv[r] = c < ncol ? qsc[(size_t)(tk0 + c / G) * a.nh + (size_t)kvh * G + c % G] : 0.0f; }
#pragma unroll
      for (int pt = 0; pt < 4; ++pt)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          const h8v Bk = nib8_f16(kw[pt][b]);
          const f4v z = {0.0f, 0.0f, 0.0f, 0.0f};
          const f4v d = __builtin_amdgcn_mfma_f32_16x16x32_f16(qa[b][1], Bk, __builtin_amdgcn_mfma_f32_16x16x32_f16(qa[b][0], Bk, z, 0, 0, 0), 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 4; ++r) D[pt][r] = fmaf(ksc[pt][b], d[r], D[pt][r]);
        }
      // register r of tile pt: column 4*lg + r, position 16*pt + li
#pragma unroll
      for (int pt = 0; pt < 4; ++pt)
#pragma unroll
        for (int r = 0; r < 4; ++r) if (4 * lg + r < ncol) red[((size_t)dq * CH + pw * 64 + 16 * pt + li) * NC + 4 * lg + r] = D[pt][r] * qinv[r];
    }
    PYRE_TS(2);
    __syncthreads(); PYRE_TS(3);
    softmax_phase(); PYRE_TS(4);
    {
      // 4-bit values on the f16 matrix cores, 32 positions x 16 dims a step.  A = the weights times the position's block
      // scale times a power of two of the wave (the largest scale lands in [2^13, 2^14)), as two f16 numbers h1 + h2
      // (rounded towards zero; row = column of the pass); B = the values, a lane's eight positions of one dim.
      float vm = wave_max(fmaxf(vsl[0], vsl[1]));
      int E = 0;
      if (vm > 0.0f && vm < INFINITY) { E = 140 - (int)((__float_as_uint(vm) >> 23) & 0xFF); E = E > 100 ? 100 : E; }
      const float up = __uint_as_float((uint32_t)(127 + E) << 23), dn = __uint_as_float((uint32_t)(127 - E) << 23);
      f4v Dv[2][2];
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int m = 0; m < 2; ++m) Dv[b][m] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
      const h2v off = {(_Float16)1032.0f, (_Float16)1032.0f};
      const int bsh = 8 * (li >> 2);
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        float ev[8];
        { const float4* e4 = (const float4*)&sc[li < NC ? li : 0][pw * 64 + 32 * g + 8 * lg];
          const float4 e0 = e4[0], e1 = e4[1]; const bool on = li < ncol;
          ev[0] = on ? e0.x : 0.0f; ev[1] = on ? e0.y : 0.0f; ev[2] = on ? e0.z : 0.0f; ev[3] = on ? e0.w : 0.0f; ev[4] = on ? e1.x : 0.0f; ev[5] = on ? e1.y : 0.0f; ev[6] = on ? e1.z : 0.0f; ev[7] = on ? e1.w : 0.0f; }
        const int vs_bits = __float_as_int(vsl[g] * up);
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          struct U4 { uint32_t v[4]; } ah, al, b0, b1;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float s0 = __int_as_float(b == 0 ? row_bcast<2 * 0>(vs_bits, q) : row_bcast<8>(vs_bits, q)), s1 = __int_as_float(b == 0 ? row_bcast<1>(vs_bits, q) : row_bcast<9>(vs_bits, q));
            const float x0 = ev[2 * q] * s0, x1 = ev[2 * q + 1] * s1;
            const auto h = __builtin_amdgcn_cvt_pkrtz(x0, x1);
            const auto l = __builtin_amdgcn_cvt_pkrtz(x0 - (float)h[0], x1 - (float)h[1]);
            ah.v[q] = __builtin_bit_cast(uint32_t, h); al.v[q] = __builtin_bit_cast(uint32_t, l);
            const uint32_t y = (((vw[g][b][2 * q] >> bsh) & 0xFFu) | (((vw[g][b][2 * q + 1] >> bsh) & 0xFFu) << 16)) ^ 0x00880088u;
            b0.v[q] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2v, (y & 0x000F000Fu) | 0x64006400u) - off);
            b1.v[q] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2v, ((y >> 4) & 0x000F000Fu) | 0x64006400u) - off);
          }
          const h8v A1 = __builtin_bit_cast(h8v, ah), A2 = __builtin_bit_cast(h8v, al), B0 = __builtin_bit_cast(h8v, b0), B1 = __builtin_bit_cast(h8v, b1);
          Dv[b][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A2, B0, __builtin_amdgcn_mfma_f32_16x16x32_f16(A1, B0, Dv[b][0], 0, 0, 0), 0, 0, 0);
          Dv[b][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A2, B1, __builtin_amdgcn_mfma_f32_16x16x32_f16(A1, B1, Dv[b][1], 0, 0, 0), 0, 0, 0);
        }
      }
      // register r of (b, m): column 4*lg + r, dim dq*64 + b*32 + 8*(li & 3) + 2*(li >> 2) + m
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
          for (int r = 0; r < 4; ++r) if (4 * lg + r < ncol) red[((size_t)pw * NC + 4 * lg + r) * HD + dq * 64 + b * 32 + 8 * (li & 3) + 2 * (li >> 2) + m] = Dv[b][m][r] * dn;
    }
  } else {
    PYRE_TS(1);
    {
      f4v D[4];
#pragma unroll
      for (int pt = 0; pt < 4; ++pt) D[pt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
      if (active) {
        float B[16];
        if (li < ncol) {
          const float4* q4 = (const float4*)(qbuf + ((size_t)(tk0 + ctok) * a.nh + (size_t)kvh * G + chead) * HD + dq * 64 + 16 * lg);
#pragma unroll
          for (int j = 0; j < 4; ++j) { float4 v = q4[j]; B[4 * j] = v.x; B[4 * j + 1] = v.y; B[4 * j + 2] = v.z; B[4 * j + 3] = v.w; }
        } else {
#pragma unroll
          for (int s = 0; s < 16; ++s) B[s] = 0.0f;
        }
        // one descriptor at the wave's 64-position block, one offset per lane; positions past the view (the last chunk)
        // read what the cache holds there, and their scores are discarded
        float A[4][16];
        const __amdgpu_buffer_rsrc_t rkf = __builtin_amdgcn_make_buffer_rsrc((void*)(kv.kf + (size_t)(wbase >> 6) * row * 64), 0, 0xFFFFFFFF, 0x00020000);
        const int kf_off = ((kvh * HD + dq * 64 + 16 * lg) * 64 + li) * 4;
#pragma unroll
        for (int pt = 0; pt < 4; ++pt)
#pragma unroll
          for (int s = 0; s < 16; ++s) A[pt][s] = __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(rkf, kf_off, (s * 64 + 16 * pt) * 4, 0));
#pragma unroll
        for (int s = 0; s < 16; ++s)
#pragma unroll
          for (int pt = 0; pt < 4; ++pt) D[pt] = __builtin_amdgcn_mfma_f32_16x16x4f32(A[pt][s], B[s], D[pt], 0, 0, 0);
        if (li < ncol) {
#pragma unroll
          for (int pt = 0; pt < 4; ++pt)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[((size_t)dq * CH + pw * 64 + 16 * pt + 4 * lg + r) * NC + li] = D[pt][r];
        }
      } else if (li < ncol) {          // a wave past the view: its positions carry no weight, their scores are read all the same
#pragma unroll
        for (int pt = 0; pt < 4; ++pt)
#pragma unroll
          for (int r = 0; r < 4; ++r) red[((size_t)dq * CH + pw * 64 + 16 * pt + 4 * lg + r) * NC + li] = 0.0f;
      }
    }
    // f32 values: requested now, while the scores are being normalised (the keys' registers are free again; __syncthreads
    // waits for outstanding loads, so the round trip is paid at the first barrier of the softmax phase instead of after the last)
    float4 vf4[16];
    if (active) {
      const __amdgpu_buffer_rsrc_t rvf = __builtin_amdgcn_make_buffer_rsrc((void*)(kv.vf + (size_t)wbase * row), 0, 0xFFFFFFFF, 0x00020000);
      const int vf_off = (kvh * HD + dq * 64 + 4 * li) * 4, last = n - 1 - wbase;
#pragma unroll
      for (int s = 0; s < 16; ++s) {          // positions past the view carry weight zero; their address is clamped
        const auto v = __builtin_amdgcn_raw_buffer_load_b128(rvf, vf_off + min(4 * s + lg, last) * (row * 4), 0, 0);
        vf4[s] = make_float4(__int_as_float(v[0]), __int_as_float(v[1]), __int_as_float(v[2]), __int_as_float(v[3]));
      }
    }
    PYRE_TS(2);
    __syncthreads(); PYRE_TS(3);
    softmax_phase(); PYRE_TS(4);
    {
      f4v D[4];
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) D[dt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
      if (active) {
        float B[16];
#pragma unroll
        for (int s = 0; s < 16; ++s) B[s] = li < ncol ? sc[li < NC ? li : 0][pw * 64 + 4 * s + lg] : 0.0f;
#pragma unroll
        for (int s = 0; s < 16; ++s) {
          const float A[4] = {vf4[s].x, vf4[s].y, vf4[s].z, vf4[s].w};
#pragma unroll
          for (int dt = 0; dt < 4; ++dt) D[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(A[dt], B[s], D[dt], 0, 0, 0);
        }
      }
      if (li < ncol) {
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
          for (int r = 0; r < 4; ++r) red[((size_t)pw * NC + li) * HD + dq * 64 + 4 * (4 * lg + r) + dt] = D[dt][r];
      }
    }
  }
  PYRE_TS(5);
  __syncthreads(); PYRE_TS(6);
  for (int i = tid; i < ncol * HD; i += NT) {
    const int c = i / HD, dd = i % HD, tk = tk0 + c / G, g = c % G;
    float o = red[((size_t)0 * NC + c) * HD + dd];
#pragma unroll
    for (int q = 1; q < NPW; ++q) o += red[((size_t)q * NC + c) * HD + dd];
    part_o[(((size_t)tk * a.nh + (size_t)kvh * G + g) * max_chunks + chunk) * HD + dd] = o;
  }
  if (tid < ncol) {
    float l = wsum[0][tid]; for (int q = 1; q < NPW; ++q) l += wsum[q][tid];
    float* ml = part_ml + (((size_t)(tk0 + tid / G) * a.nh + (size_t)kvh * G + tid % G) * max_chunks + chunk) * 2;
    float mm = wmax[0][tid]; for (int q = 1; q < NPW; ++q) mm = fmaxf(mm, wmax[q][tid]);
    ml[0] = mm; ml[1] = l;
  }
#ifdef PYRE_PHASE_TS
  PYRE_TS(7);
  if (tid == 0 && kvh == 0 && blockIdx.z == 0 && (chunk == 0 || chunk == (n - 1) / CH)) { for (int q_ = 0; q_ < 8; ++q_) attn_ts[(chunk == 0 ? 0 : 8) + q_] = ts_[q_]; }
  if (tid == 0 && blockIdx.z == 0) { const unsigned w_ = blockIdx.y * gridDim.x + blockIdx.x; if (w_ < 4096) { for (int q_ = 0; q_ < 8; ++q_) attn_wg[10 * w_ + q_] = ts_[q_];
    attn_wg[10 * w_ + 8] = ((unsigned long long)__builtin_amdgcn_s_getreg(20 | (31 << 11)) << 32) | (unsigned)__builtin_amdgcn_s_getreg(4 | (31 << 11)); attn_wg[10 * w_ + 9] = ((unsigned long long)kvh << 32) | (unsigned)chunk; } }
#endif
}

// The same kernel over a position list: entry i of plist[ti] (pcount[ti] entries, ascending positions) takes the place of
// position i; pcount[ti] < 0 means every visible position (the list is not read).  Listed positions are scattered over
// the packed and the f32 part of the cache, so the choice between them is made per lane, not per wave.
template <int HD, int G>
__global__ __launch_bounds__(256 * PYRE_ATTN_NPW) void k_attn_decode_sel(AttnDev a, KvDev kv, const float* __restrict__ qbuf, int start, const int* __restrict__ posp, float* __restrict__ part_o, float* __restrict__ part_ml, int max_chunks,
                                                                         const int* __restrict__ plist, const int* __restrict__ pcount, int list_stride) {
  static_assert(HD == 256, "the wave layout assumes 4 x 64 head dims");
  constexpr int NPW = PYRE_ATTN_NPW, CH = PYRE_ATTN_CHUNK, NT = 256 * NPW;
  __shared__ float red[4 * CH * G];
  __shared__ float sc[CH][G];
  __shared__ float wmax[NPW][G], wsum[NPW][G], cm[G];
  const int lin = (int)blockIdx.x + (int)gridDim.x * (int)blockIdx.y;          // dispatch order as in k_attn_decode
  const int chunk = (int)gridDim.x - 1 - lin / (int)gridDim.y, kvh = lin % (int)gridDim.y, ti = blockIdx.z, tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), pw = wave % NPW, dq = wave / NPW;
  if (posp) start = *posp;
  const int n = start + ti + 1, cnt = pcount[ti];
  const bool listed = cnt >= 0; const int ne = listed ? cnt : n;       // entries to attend to
  if (chunk * CH >= ne) return;
  const int* list = plist + (size_t)ti * list_stride;
  const int pb = (int)((a.kv_bits == 4 && n > a.kv_recent + 64) ? ((n - a.kv_recent) / 64) * 64 : 0);
  const int wbase = chunk * CH + pw * 64;
  const bool valid = wbase + lane < ne, active = wbase < ne;
  const float scale = 1.0f / sqrtf((float)HD);
  const int li = lane & 15, lg = lane >> 4;
  const int row = a.nkv * HD;
  auto pos_of = [&](int i) { int ii = min(i, ne - 1); return listed ? list[ii] : ii; };
  {
    f4v D[4];
#pragma unroll
    for (int pt = 0; pt < 4; ++pt) D[pt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
    if (active) {
      float B[16];
      if (li < G) {
        const float4* q4 = (const float4*)(qbuf + ((size_t)ti * a.nh + (size_t)kvh * G + li) * HD + dq * 64 + 16 * lg);
#pragma unroll
        for (int j = 0; j < 4; ++j) { float4 v = q4[j]; B[4 * j] = v.x; B[4 * j + 1] = v.y; B[4 * j + 2] = v.z; B[4 * j + 3] = v.w; }
      } else {
#pragma unroll
        for (int s = 0; s < 16; ++s) B[s] = 0.0f;
      }
      float A[4][16];
      // Whether a position is read from the 4-bit or the f32 part is a per-lane fact, but almost every wave is all of one
      // kind (old selected blocks, or the tail): those take a branch the whole wave agrees on, with all loads in flight
      // at once; only a wave that straddles the boundary decides lane by lane.
      size_t pp[4]; bool lp = true, lf = true;
#pragma unroll
      for (int pt = 0; pt < 4; ++pt) { pp[pt] = (size_t)pos_of(wbase + 16 * pt + li); lp = lp && (int)pp[pt] < pb; lf = lf && (int)pp[pt] >= pb; }
      if (__all(lp)) {
        uint32_t kw[4][2]; float ksc[4];
#pragma unroll
        for (int pt = 0; pt < 4; ++pt) {
          kw[pt][0] = kv.kq[kv_blk((size_t)kvh * (HD / 8) + dq * 8 + 2 * lg, (size_t)a.nkv * (HD / 8), pp[pt])]; kw[pt][1] = kv.kq[kv_blk((size_t)kvh * (HD / 8) + dq * 8 + 2 * lg + 1, (size_t)a.nkv * (HD / 8), pp[pt])];
          ksc[pt] = kv.ks[kv_blk((size_t)kvh * (HD / 32) + dq * 2 + (lg >> 1), (size_t)a.nkv * (HD / 32), pp[pt])];
        }
#pragma unroll
        for (int pt = 0; pt < 4; ++pt)
#pragma unroll
          for (int s = 0; s < 16; ++s) A[pt][s] = nib_val(kw[pt][s >> 3], s & 7) * ksc[pt];
      } else if (__all(lf)) {
#pragma unroll
        for (int pt = 0; pt < 4; ++pt)
#pragma unroll
          for (int s = 0; s < 16; ++s) A[pt][s] = kv.kf[kv_blk((size_t)kvh * HD + dq * 64 + 16 * lg + s, (size_t)a.nkv * HD, pp[pt])];
      } else {
#pragma unroll
        for (int pt = 0; pt < 4; ++pt) {
          if ((int)pp[pt] < pb) {
            uint32_t k0 = kv.kq[kv_blk((size_t)kvh * (HD / 8) + dq * 8 + 2 * lg, (size_t)a.nkv * (HD / 8), pp[pt])], k1 = kv.kq[kv_blk((size_t)kvh * (HD / 8) + dq * 8 + 2 * lg + 1, (size_t)a.nkv * (HD / 8), pp[pt])];
            float ksc = kv.ks[kv_blk((size_t)kvh * (HD / 32) + dq * 2 + (lg >> 1), (size_t)a.nkv * (HD / 32), pp[pt])];
#pragma unroll
            for (int s = 0; s < 16; ++s) A[pt][s] = nib_val(s < 8 ? k0 : k1, s & 7) * ksc;
          } else {
#pragma unroll
            for (int s = 0; s < 16; ++s) A[pt][s] = kv.kf[kv_blk((size_t)kvh * HD + dq * 64 + 16 * lg + s, (size_t)a.nkv * HD, pp[pt])];
          }
        }
      }
#pragma unroll
      for (int s = 0; s < 16; ++s)
#pragma unroll
        for (int pt = 0; pt < 4; ++pt) D[pt] = __builtin_amdgcn_mfma_f32_16x16x4f32(A[pt][s], B[s], D[pt], 0, 0, 0);
    }
    if (li < G) {
#pragma unroll
      for (int pt = 0; pt < 4; ++pt)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[((size_t)dq * CH + pw * 64 + 16 * pt + 4 * lg + r) * G + li] = D[pt][r];
    }
  }
  __syncthreads();
  constexpr int GH = (G + 3) / 4;
  const int pos = pw * 64 + lane;
  float sv[GH];
#pragma unroll
  for (int gi = 0; gi < GH; ++gi) {
    const int g = dq + 4 * gi; sv[gi] = -INFINITY;
    if (g < G) {
      float v = ((red[((size_t)0 * CH + pos) * G + g] + red[((size_t)1 * CH + pos) * G + g]) + red[((size_t)2 * CH + pos) * G + g]) + red[((size_t)3 * CH + pos) * G + g];
      sv[gi] = valid ? v * scale : -INFINITY;
      const float m = wave_max(sv[gi]);
      if (lane == 0) wmax[pw][g] = m;
    }
  }
  __syncthreads();
  if (tid < G) { float mm = wmax[0][tid]; for (int q = 1; q < NPW; ++q) mm = fmaxf(mm, wmax[q][tid]); cm[tid] = mm; }
  __syncthreads();
#pragma unroll
  for (int gi = 0; gi < GH; ++gi) {
    const int g = dq + 4 * gi;
    if (g < G) {
      float e = valid ? expf(sv[gi] - cm[g]) : 0.0f; sc[pos][g] = e;
      const float l = wave_sum(e);
      if (lane == 0) wsum[pw][g] = l;
    }
  }
  __syncthreads();
  {
    f4v D[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) D[dt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
    if (active) {
      float A[4][16];
      size_t pg[16]; bool lp = true, lf = true;             // entries past the list carry weight zero; their position is clamped
#pragma unroll
      for (int s = 0; s < 16; ++s) { pg[s] = (size_t)pos_of(wbase + 4 * s + lg); lp = lp && (int)pg[s] < pb; lf = lf && (int)pg[s] >= pb; }
      if (__all(lp)) {
        uint32_t vw[16]; float vsc[16];
#pragma unroll
        for (int s = 0; s < 16; ++s) {
          vw[s] = kv.vq[pg[s] * (row / 8) + (size_t)kvh * (HD / 8) + dq * 8 + (li >> 1)];
          vsc[s] = kv.vs[pg[s] * (row / 32) + (size_t)kvh * (HD / 32) + dq * 2 + (li >> 3)];
        }
#pragma unroll
        for (int s = 0; s < 16; ++s) {
          const uint32_t hw = vw[s] >> (16 * (li & 1));
#pragma unroll
          for (int dt = 0; dt < 4; ++dt) A[dt][s] = nib_val(hw, dt) * vsc[s];
        }
      } else if (__all(lf)) {
#pragma unroll
        for (int s = 0; s < 16; ++s) {
          float4 v = *(const float4*)(kv.vf + pg[s] * row + (size_t)kvh * HD + dq * 64 + 4 * li);
          A[0][s] = v.x; A[1][s] = v.y; A[2][s] = v.z; A[3][s] = v.w;
        }
      } else {
#pragma unroll
        for (int s = 0; s < 16; ++s) {
          if ((int)pg[s] < pb) {
            const uint32_t vw = kv.vq[pg[s] * (row / 8) + (size_t)kvh * (HD / 8) + dq * 8 + (li >> 1)];
            const float vsc = kv.vs[pg[s] * (row / 32) + (size_t)kvh * (HD / 32) + dq * 2 + (li >> 3)];
            const uint32_t hw = vw >> (16 * (li & 1));
#pragma unroll
            for (int dt = 0; dt < 4; ++dt) A[dt][s] = nib_val(hw, dt) * vsc;
          } else {
            float4 v = *(const float4*)(kv.vf + pg[s] * row + (size_t)kvh * HD + dq * 64 + 4 * li);
            A[0][s] = v.x; A[1][s] = v.y; A[2][s] = v.z; A[3][s] = v.w;
          }
        }
      }
      float B[16];
#pragma unroll
      for (int s = 0; s < 16; ++s) B[s] = li < G ? sc[pw * 64 + 4 * s + lg][li < G ? li : 0] : 0.0f;
#pragma unroll
      for (int s = 0; s < 16; ++s)
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) D[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(A[dt][s], B[s], D[dt], 0, 0, 0);
    }
    if (li < G) {
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[((size_t)pw * G + li) * HD + dq * 64 + 4 * (4 * lg + r) + dt] = D[dt][r];
    }
  }
  __syncthreads();
  for (int i = tid; i < G * HD; i += NT) {
    int g = i / HD, dd = i % HD;
    float o = red[((size_t)0 * G + g) * HD + dd];
#pragma unroll
    for (int q = 1; q < NPW; ++q) o += red[((size_t)q * G + g) * HD + dd];
    part_o[(((size_t)ti * a.nh + (size_t)kvh * G + g) * max_chunks + chunk) * HD + dd] = o;
  }
  if (tid < G) {
    float l = wsum[0][tid]; for (int q = 1; q < NPW; ++q) l += wsum[q][tid];
    float* ml = part_ml + (((size_t)ti * a.nh + (size_t)kvh * G + tid) * max_chunks + chunk) * 2;
    ml[0] = cm[tid]; ml[1] = l;
  }
}

// grid (nh, t, HD/16), 256 threads: merge the chunk partials (log-sum-exp), normalise, multiply by sigmoid(gate).
// Thread (grp, dim) adds the chunks grp, grp+16, ... in ascending order; the sixteen groups are then added in order.
// A workgroup owns 16 dimensions of a head -- the partial outputs are most of what a long context makes this kernel read,
// and a compute unit fetches them no faster than about 20 GB/s, so they are spread over nh * 16 workgroups -- and goes
// through the chunks 320 at a time: the 20 partial outputs a thread needs of such a tile do not depend on the maximum,
// so the first tile's are fetched at the start, together with the (max, sum) pairs and the gate; thread c of the tile
// (and again thread c - 256 for the last 64) then leaves exp(max_c - M) and sum_c in shared memory for everybody.  Up to
// 320 chunks (40 960 positions) the whole merge is one memory round trip -- the step after a 32 768-token prompt has 257.
template <int HD>
__global__ __launch_bounds__(256) void k_attn_combine(AttnDev a, const float* __restrict__ qkv, int stride, int start, const int* __restrict__ posp, const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                      int max_chunks, float* __restrict__ out, const int* __restrict__ pcount) {
  constexpr int CB = 320, DW = PYRE_ATTN_CDIMS, NG = 256 / DW, B = CB / NG;
  PYRE_TS_VARS PYRE_TS(0);
  __shared__ float wmax[4]; __shared__ float so[NG][DW]; __shared__ float sl[NG]; __shared__ float fs[CB], ls[CB];
  if (posp) start = *posp;
  const int h = blockIdx.x, ti = blockIdx.y, tid = threadIdx.x, grp = tid / DW, dl = tid % DW, dd = blockIdx.z * DW + dl;
  int n = start + ti + 1; if (pcount && pcount[ti] >= 0) n = pcount[ti];        // a position list: its entries are what the chunks covered
  const int nc = (n + PYRE_ATTN_CHUNK - 1) / PYRE_ATTN_CHUNK;
  const float* ml = part_ml + ((size_t)ti * a.nh + h) * max_chunks * 2;
  const float* po = part_o + ((size_t)ti * a.nh + h) * max_chunks * HD;
  const float gate = grp == 0 ? qkv[(size_t)ti * stride + (size_t)h * 2 * HD + HD + dd] : 0.0f;          // fetched with the partials, not after them
  float pv[B];
#pragma unroll
  for (int i = 0; i < B; ++i) pv[i] = nc > 0 ? po[(size_t)min(grp + NG * i, nc - 1) * HD + dd] : 0.0f;
  float m0 = -INFINITY, l0 = 0.0f, m1 = -INFINITY, l1 = 0.0f;          // the tile's chunks tid and (threads below 64) 256 + tid
  if (tid < nc) { m0 = ml[2 * tid]; l0 = ml[2 * tid + 1]; }
  if (tid < CB - 256 && 256 + tid < nc) { m1 = ml[2 * (256 + tid)]; l1 = ml[2 * (256 + tid) + 1]; }
  float M = m0; for (int c = tid + 256; c < nc; c += 256) M = fmaxf(M, ml[2 * c]);
  M = wave_max(M);
  if ((tid & 63) == 0) wmax[tid >> 6] = M;
  __syncthreads();
  M = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
  float L = 0.0f, o = 0.0f;
  for (int cb = 0; cb < nc; cb += CB) {
    if (cb > 0) {
      __syncthreads();
#pragma unroll
      for (int i = 0; i < B; ++i) pv[i] = po[(size_t)min(cb + grp + NG * i, nc - 1) * HD + dd];
      m0 = -INFINITY; l0 = 0.0f; if (cb + tid < nc) { m0 = ml[2 * (cb + tid)]; l0 = ml[2 * (cb + tid) + 1]; }
      m1 = -INFINITY; l1 = 0.0f; if (tid < CB - 256 && cb + 256 + tid < nc) { m1 = ml[2 * (cb + 256 + tid)]; l1 = ml[2 * (cb + 256 + tid) + 1]; }
    }
    fs[tid] = expf(m0 - M); ls[tid] = l0;
    if (tid < CB - 256) { fs[256 + tid] = expf(m1 - M); ls[256 + tid] = l1; }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < B; ++i) if (cb + grp + NG * i < nc) { const float f = fs[grp + NG * i]; L = fmaf(ls[grp + NG * i], f, L); o = fmaf(pv[i], f, o); }
  }
  so[grp][dl] = o; if (dl == 0) sl[grp] = L;
  __syncthreads();
  if (grp == 0) {
    o = so[0][dl]; L = sl[0];
#pragma unroll
    for (int g = 1; g < NG; ++g) { o += so[g][dl]; L += sl[g]; }
    const float ov = (o / L) * a_sigm(gate);
    out[((size_t)ti * a.nh + h) * HD + dd] = ov;
  }
  PYRE_TS(1); PYRE_TS(2); PYRE_TS(3); PYRE_TS(4); PYRE_TS(5); PYRE_TS(6); PYRE_TS(7); PYRE_TS_FLUSH(attn_ts, 16);
}

size_t pyre_kv_bytes(const AttnDev& a, int cap) {
  size_t row = (size_t)a.nkv * a.hd, c = cap;
  return 6 * 256 + c * row * 4 * 2 + c * row / 8 * 4 * 2 + c * row / 32 * 4 * 2;
}
void pyre_kv_carve(const AttnDev& a, int cap, void* base, KvDev* kv) {
  uint8_t* p = (uint8_t*)base; auto take = [&](size_t n) { void* r = p; p += (n + 255) & ~(size_t)255; return r; };
  size_t row = (size_t)a.nkv * a.hd, c = cap;
  kv->kf = (float*)take(c * row * 4); kv->vf = (float*)take(c * row * 4); kv->kq = (uint32_t*)take(c * row / 8 * 4); kv->ks = (float*)take(c * row / 32 * 4);
  kv->vq = (uint32_t*)take(c * row / 8 * 4); kv->vs = (float*)take(c * row / 32 * 4); kv->cap = cap;
}
size_t pyre_attn_work_bytes(const AttnDev& a, int cap) {
  size_t mc = ((size_t)cap + PYRE_ATTN_CHUNK - 1) / PYRE_ATTN_CHUNK;
  return 5 * 256 + 4 * (2 * 8 * (size_t)a.nh * a.hd + 8 * (size_t)a.nh + 8 * (size_t)a.nh * mc * a.hd + 8 * (size_t)a.nh * mc * 2);
}
void pyre_attn_work_carve(const AttnDev& a, int cap, void* base, AttnWork* w) {
  uint8_t* p = (uint8_t*)base; auto take = [&](size_t n) { void* r = p; p += (n + 255) & ~(size_t)255; return r; };
  size_t mc = ((size_t)cap + PYRE_ATTN_CHUNK - 1) / PYRE_ATTN_CHUNK;
  w->q = (float*)take(4 * 8 * (size_t)a.nh * a.hd); w->qh = (uint16_t*)take(2 * 2 * 8 * (size_t)a.nh * a.hd); w->qsc = (float*)take(4 * 8 * (size_t)a.nh); w->part_o = (float*)take(4 * 8 * (size_t)a.nh * mc * a.hd); w->part_ml = (float*)take(4 * 8 * (size_t)a.nh * mc * 2); w->max_chunks = (int)mc;
}

template <int G> static void launch_decode(pyre_ctx* ctx, const AttnDev& a, const KvDev& kv, const AttnWork& w, int start, int t, const int* posp, const QsaWork* qw) {
  int n = start + t, chunks = posp ? w.max_chunks : (n + PYRE_ATTN_CHUNK - 1) / PYRE_ATTN_CHUNK;      // device-side position: cover the whole cache, surplus workgroups leave at once
  if (!qw) {          // tokens that share a pass over the cache: as many as the 16 columns hold, one when the 4-bit boundary moves inside the window
    int tp = 16 / G > 8 ? 8 : 16 / G;
    if (posp || pyre_packed_boundary((size_t)start + 1, a.kv_bits, a.kv_recent) != pyre_packed_boundary((size_t)start + t, a.kv_bits, a.kv_recent)) tp = 1;
    if (tp == 1 || t == 1) hipLaunchKernelGGL((k_attn_decode<256, G, G>), dim3(chunks, a.nkv, t), dim3(256 * PYRE_ATTN_NPW), 0, ctx->stream, a, kv, w.q, w.qh, w.qsc, start, posp, w.part_o, w.part_ml, w.max_chunks, t, 1);
    else hipLaunchKernelGGL((k_attn_decode<256, G, 16>), dim3(chunks, a.nkv, (t + tp - 1) / tp), dim3(256 * PYRE_ATTN_NPW), 0, ctx->stream, a, kv, w.q, w.qh, w.qsc, start, posp, w.part_o, w.part_ml, w.max_chunks, t, tp);
    return; }
  // a token attends either to all of its n <= budget + ratio - 1 visible positions or to a list: never to more than list_stride entries
  { int lc = (qw->list_stride + PYRE_ATTN_CHUNK - 1) / PYRE_ATTN_CHUNK; if (chunks > lc) chunks = lc; }
  hipLaunchKernelGGL((k_attn_decode_sel<256, G>), dim3(chunks, a.nkv, t), dim3(256 * PYRE_ATTN_NPW), 0, ctx->stream, a, kv, w.q, start, posp, w.part_o, w.part_ml, w.max_chunks, qw->plist, qw->pcount, qw->list_stride);
}

int pyre_attn_launch(pyre_ctx* ctx, const AttnDev& a, const KvDev& kv, const AttnWork& w, const float* qkv, int stride, int start, int t, int* packed_done, float* out, const int* posp) {
  return pyre_attn_launch_sel(ctx, a, kv, w, qkv, stride, start, t, packed_done, out, posp, nullptr);
}
int pyre_attn_launch_sel(pyre_ctx* ctx, const AttnDev& a, const KvDev& kv, const AttnWork& w, const float* qkv, int stride, int start, int t, int* packed_done, float* out, const int* posp, const QsaWork* qw, int part) {
  if (a.hd != 256) return pyre_fail(ctx, PYRE_E_SHAPE, "attention: head dim %d unsupported (256 only)", a.hd);
  if (a.nkv < 1 || a.nh % a.nkv) return pyre_fail(ctx, PYRE_E_SHAPE, "attention: %d query heads over %d kv heads", a.nh, a.nkv);
  int G = a.nh / a.nkv; if (G != 1 && G != 2 && G != 4 && G != 8) return pyre_fail(ctx, PYRE_E_SHAPE, "attention: group size %d unsupported (1, 2, 4, 8)", G);
  if (t < 1 || t > 8) return pyre_fail(ctx, PYRE_E_ARG, "attention: t = %d outside 1..8", t);
  if (start < 0 || start + t > kv.cap) return pyre_fail(ctx, PYRE_E_STATE, "attention: position %d exceeds the cache capacity %d", start + t, kv.cap);
  if (a.n_rot > a.hd || (a.n_rot & 1)) return pyre_fail(ctx, PYRE_E_SHAPE, "attention: n_rot %d", a.n_rot);
  // a single-token step at a device-side position: the packing check rides on the prep launch as extra blocks
  // part 1: the cache write (rotated q into w.q / qh / qsc, K and V into the cache, packing); part 2: the attention pass over
  // the cache and the merge, which read only what part 1 of this and of earlier windows has written (w.q* must then be this
  // window's own until part 2 has run); 0: both
  if (part < 0 || part > 2 || (part && posp)) return pyre_fail(ctx, PYRE_E_ARG, "attention: part %d", part);
  const int nwin = ctx->batch_n;          // part 1 for that many consecutive windows of t tokens in one launch (ctx->batch_stride / batch_stride2: the windows' projections / query buffers apart)
  if (nwin > 1 && (part != 1 || qw || start + nwin * t > kv.cap)) return pyre_fail(ctx, PYRE_E_ARG, "attention: %d windows a launch (the cache write alone, dense, inside the cache)", nwin);
  const bool pack_rides = posp && t == 1 && a.kv_bits == 4;
  const int pack_blocks = pack_rides ? (64 * (a.nkv * a.hd / 32) * 2 + 255) / 256 : 0;
  if (part != 2) {
  { ProfScope ps(ctx, "attn_prep", 8.0 * t * (a.nh + 2.0 * a.nkv) * a.hd); hipLaunchKernelGGL((k_attn_prep<256>), dim3(a.nkv + a.nh + pack_blocks, t, nwin), dim3(256), 0, ctx->stream, a, kv, qkv, stride, start, posp, w.q, w.qh, w.qsc, ctx->batch_stride, ctx->batch_stride2); } PYRE_CHECK_LAUNCH(ctx);
  // pack the positions that fall below the boundary of the longest view of this call
  int pbn = (int)pyre_packed_boundary((size_t)start + (size_t)nwin * t, a.kv_bits, a.kv_recent);
  if (posp) {   // one 64-position packing step at most; the kernel decides from the device-side position
    if (a.kv_bits == 4 && !pack_rides) { size_t thr = (size_t)64 * (a.nkv * a.hd / 32) * 2; hipLaunchKernelGGL((k_kv_pack<256>), dim3((unsigned)((thr + 127) / 128)), dim3(128), 0, ctx->stream, a, kv, 0, 0, posp); PYRE_CHECK_LAUNCH(ctx); }
  } else if (pbn > *packed_done) {
    size_t thr = (size_t)(pbn - *packed_done) * (a.nkv * a.hd / 32) * 2;
    { ProfScope ps(ctx, "kv_pack", (double)(pbn - *packed_done) * a.nkv * a.hd * 2 * 4.625); hipLaunchKernelGGL((k_kv_pack<256>), dim3((unsigned)((thr + 127) / 128)), dim3(128), 0, ctx->stream, a, kv, *packed_done, pbn, (const int*)nullptr); } PYRE_CHECK_LAUNCH(ctx);
    *packed_done = pbn;
  }
  }
  if (part == 1) return PYRE_OK;
  double kvb = 0;
  for (int ti = 0; ti < t; ++ti) {
    double n = start + ti + 1, pb = (double)pyre_packed_boundary((size_t)n, a.kv_bits, a.kv_recent);
    if (qw && n > qw->list_stride) { double m = qw->list_stride, fp = n > 0 ? pb / n : 0; kvb += 2.0 * a.nkv * a.hd * m * (fp * 0.625 + (1 - fp) * 4.0); }     // a position list: its entries, packed in the cache's own proportion
    else kvb += 2.0 * a.nkv * a.hd * (pb * 0.625 + (n - pb) * 4.0);
  }
  { ProfScope ps(ctx, "attn_decode", kvb);
  switch (G) { case 1: launch_decode<1>(ctx, a, kv, w, start, t, posp, qw); break; case 2: launch_decode<2>(ctx, a, kv, w, start, t, posp, qw); break; case 4: launch_decode<4>(ctx, a, kv, w, start, t, posp, qw); break;
    default: launch_decode<8>(ctx, a, kv, w, start, t, posp, qw); } }
  PYRE_CHECK_LAUNCH(ctx);
  { ProfScope ps(ctx, "attn_combine", 4.0 * t * a.nh * a.hd * ((start + t + PYRE_ATTN_CHUNK - 1) / PYRE_ATTN_CHUNK + 2)); hipLaunchKernelGGL((k_attn_combine<256>), dim3(a.nh, t, 256 / PYRE_ATTN_CDIMS), dim3(256), 0, ctx->stream, a, qkv, stride, start, posp, w.part_o, w.part_ml, w.max_chunks, out, qw ? qw->pcount : (const int*)nullptr); } PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}

// K / V of positions start..start+t-1 into an f32 cache, nothing attended (the drafter's catch-up over committed cells)
int pyre_attn_append_launch(pyre_ctx* ctx, const AttnDev& a, const KvDev& kv, const AttnWork& w, const float* qkv, int stride, int start, int t) {
  if (a.hd != 256 || a.kv_bits != 0) return pyre_fail(ctx, PYRE_E_SHAPE, "attention append: head dim %d, %d-bit cache (256, f32 only)", a.hd, a.kv_bits);
  if (t < 1 || t > 8 || start < 0 || start + t > kv.cap) return pyre_fail(ctx, PYRE_E_STATE, "attention append: positions %d..%d outside the cache (%d)", start, start + t, kv.cap);
  { ProfScope ps(ctx, "attn_prep", 8.0 * t * (a.nh + 2.0 * a.nkv) * a.hd); hipLaunchKernelGGL((k_attn_prep<256>), dim3(a.nkv + a.nh, t), dim3(256), 0, ctx->stream, a, kv, qkv, stride, start, (const int*)nullptr, w.q, w.qh, w.qsc, (size_t)0, (size_t)0); } PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}

// ---- C ABI: standalone attention layer core for the block harness -----------------------------------------------------
struct pyre_attn { pyre_ctx* ctx; AttnDev dv; KvDev kv; AttnWork w; float* params; void* kvmem; void* wmem; float* io; int len, packed, cap;
                   QsaDev q{}; QsaBuf qb{}; QsaWork qw{}; void* qmem = nullptr; float* qparams = nullptr; float rope_base = 0; };

extern "C" {

int pyre_attn_create(pyre_ctx* ctx, int nh, int nkv, int hd, int n_rot, float rope_base, float eps, const float* qn, const float* kn, int kv_bits, int kv_recent, int max_ctx, pyre_attn** out) {
  if (!ctx || !out || !qn || !kn) return pyre_fail(ctx, PYRE_E_ARG, "pyre_attn_create: null argument");
  *out = nullptr;
  if (hd != 256 || nkv < 1 || nh % nkv || n_rot > hd || (n_rot & 1) || max_ctx < 1 || (kv_bits != 0 && kv_bits != 4) || kv_recent < 64) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_attn_create: unsupported geometry");
  pyre_attn* a = new pyre_attn(); a->ctx = ctx; a->len = 0; a->packed = 0; a->cap = (max_ctx + 255) / 256 * 256;
  std::vector<float> hp(2 * (size_t)hd + n_rot / 2); memcpy(hp.data(), qn, 4 * hd); memcpy(hp.data() + hd, kn, 4 * hd);
  for (int i = 0; i < n_rot / 2; ++i) hp[2 * hd + i] = powf(rope_base, -(2.0f * (float)i) / (float)n_rot);    // rope_inv, src/qn_ctx.rs:168
  a->dv = AttnDev{nullptr, nullptr, nullptr, nh, nkv, hd, n_rot, kv_bits, kv_recent, eps}; a->rope_base = rope_base;
  size_t qw = (size_t)nh * 2 * hd + 2 * (size_t)nkv * hd;
  hipError_t e = hipMalloc((void**)&a->params, hp.size() * 4);
  if (e == hipSuccess) e = hipMemcpy(a->params, hp.data(), hp.size() * 4, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMalloc(&a->kvmem, pyre_kv_bytes(a->dv, a->cap));
  if (e == hipSuccess) e = hipMalloc(&a->wmem, pyre_attn_work_bytes(a->dv, a->cap));
  if (e == hipSuccess) e = hipMalloc((void**)&a->io, 8 * (qw + (size_t)nh * hd) * 4);
  if (e != hipSuccess) { int rc = pyre_fail(ctx, PYRE_E_HIP, "pyre_attn_create: %s", hipGetErrorString(e)); delete a; return rc; }
  a->dv.qn = a->params; a->dv.kn = a->params + hd; a->dv.rope_inv = a->params + 2 * hd;
  pyre_kv_carve(a->dv, a->cap, a->kvmem, &a->kv); pyre_attn_work_carve(a->dv, a->cap, a->wmem, &a->w);
  *out = a; return PYRE_OK;
}
void pyre_attn_destroy(pyre_attn* a) { if (!a) return; (void)hipStreamSynchronize(a->ctx->stream); if (a->qmem) (void)hipFree(a->qmem); if (a->qparams) (void)hipFree(a->qparams); (void)hipFree(a->params); (void)hipFree(a->kvmem); (void)hipFree(a->wmem); (void)hipFree(a->io); delete a; }
int pyre_attn_len(const pyre_attn* a) { return a ? a->len : 0; }
int pyre_attn_truncate(pyre_ctx* ctx, pyre_attn* a, int len) { if (!a || len < 0 || len > a->len) return pyre_fail(ctx, PYRE_E_ARG, "pyre_attn_truncate: bad length"); a->len = len; return PYRE_OK; }

// Decode / verify step of one attention layer over its own cache: qkv [t][nh*2*hd + 2*nkv*hd] raw projections for the
// next t positions -> out [t][nh*hd]; the positions are appended to the cache.
int pyre_attn_decode_kv4(pyre_ctx* ctx, pyre_attn* a, const float* qkv_host, int t, float* out_host) {
  if (!ctx || !a || !qkv_host || !out_host) return pyre_fail(ctx, PYRE_E_ARG, "pyre_attn_decode_kv4: null argument");
  if (t < 1 || t > 8) return pyre_fail(ctx, PYRE_E_ARG, "pyre_attn_decode_kv4: t = %d outside 1..8", t);
  size_t qb = (size_t)a->dv.nh * 2 * a->dv.hd + 2 * (size_t)a->dv.nkv * a->dv.hd, qw = qb + (a->q.nh > 0 ? (size_t)(a->q.nh + 1) * a->q.hd : 0), ow = (size_t)a->dv.nh * a->dv.hd;
  float* qd = a->io; float* od = a->io + 8 * qw;
  PYRE_HIP(ctx, hipMemcpyAsync(qd, qkv_host, (size_t)t * qw * 4, hipMemcpyHostToDevice, ctx->stream));
  int rc = PYRE_OK;
  if (a->q.nh > 0 && (rc = pyre_qsa_launch(ctx, a->q, a->dv, a->qb, a->qw, qd, (int)qw, (int)qb, a->len, t, nullptr))) return rc;
  rc = pyre_attn_launch_sel(ctx, a->dv, a->kv, a->w, qd, (int)qw, a->len, t, &a->packed, od, nullptr, a->q.nh > 0 ? &a->qw : nullptr); if (rc) return rc;
  a->len += t;
  PYRE_HIP(ctx, hipMemcpyAsync(out_host, od, (size_t)t * ow * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}
// Test / harness access: load n positions of already-normalised keys and values (row-major [n][nkv*hd]) as the cache
// content, and read the f32 rows back.
int pyre_attn_load_cache(pyre_ctx* ctx, pyre_attn* a, const float* k_host, const float* v_host, int n) {
  if (!ctx || !a || !k_host || !v_host || n < 0 || n > a->cap) return pyre_fail(ctx, PYRE_E_ARG, "pyre_attn_load_cache: bad argument");
  size_t row = (size_t)a->dv.nkv * a->dv.hd; std::vector<float> kt(row * a->cap, 0.0f);
  for (int p = 0; p < n; ++p) for (size_t c = 0; c < row; ++c) kt[kv_blk(c, row, p)] = k_host[(size_t)p * row + c];
  PYRE_HIP(ctx, hipMemcpyAsync(a->kv.kf, kt.data(), kt.size() * 4, hipMemcpyHostToDevice, ctx->stream));
  PYRE_HIP(ctx, hipMemcpyAsync(a->kv.vf, v_host, (size_t)n * row * 4, hipMemcpyHostToDevice, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
  a->len = n; a->packed = 0;
  int pbn = (int)pyre_packed_boundary((size_t)n, a->dv.kv_bits, a->dv.kv_recent);
  if (pbn > 0) { size_t thr = (size_t)pbn * (row / 32) * 2; hipLaunchKernelGGL((k_kv_pack<256>), dim3((unsigned)((thr + 127) / 128)), dim3(128), 0, ctx->stream, a->dv, a->kv, 0, pbn, (const int*)nullptr); PYRE_CHECK_LAUNCH(ctx); a->packed = pbn; PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); }
  return PYRE_OK;
}
int pyre_attn_read_cache(pyre_ctx* ctx, pyre_attn* a, float* k_host, float* v_host) {
  if (!ctx || !a || !k_host || !v_host) return pyre_fail(ctx, PYRE_E_ARG, "pyre_attn_read_cache: null argument");
  size_t row = (size_t)a->dv.nkv * a->dv.hd; std::vector<float> kt(row * a->cap);
  PYRE_HIP(ctx, hipMemcpyAsync(kt.data(), a->kv.kf, kt.size() * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipMemcpyAsync(v_host, a->kv.vf, (size_t)a->len * row * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
  for (int p = 0; p < a->len; ++p) for (size_t c = 0; c < row; ++c) k_host[(size_t)p * row + c] = kt[kv_blk(c, row, p)];
  return PYRE_OK;
}
// Attaches a QSA indexer to the block (before any position is decoded): rows passed to pyre_attn_decode_kv4 then carry
// [.. | index queries nh*hd | index key hd] after the q/k/v projections.
int pyre_attn_set_indexer(pyre_ctx* ctx, pyre_attn* a, int idx_nh, int idx_hd, int idx_ratio, int idx_budget, const float* iqn_host, const float* ikn_host) {
  if (!ctx || !a || !iqn_host || !ikn_host) return pyre_fail(ctx, PYRE_E_ARG, "pyre_attn_set_indexer: null argument");
  if (a->len != 0 || a->q.nh != 0) return pyre_fail(ctx, PYRE_E_STATE, "pyre_attn_set_indexer: the block already holds positions or an indexer");
  if (idx_nh < 1 || idx_hd < 64 || idx_hd % 64 || idx_hd > 1024 || idx_hd < a->dv.n_rot || idx_ratio < 1 || idx_budget < idx_ratio || idx_budget % idx_ratio) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_attn_set_indexer: unsupported geometry");
  QsaDev q{nullptr, nullptr, idx_nh, idx_hd, idx_ratio, idx_budget};
  size_t bb = (pyre_qsa_buf_bytes(q, a->cap) + 255) & ~(size_t)255, wb = pyre_qsa_work_bytes(q, a->cap);
  size_t qw = (size_t)a->dv.nh * 2 * a->dv.hd + 2 * (size_t)a->dv.nkv * a->dv.hd + (size_t)(idx_nh + 1) * idx_hd;
  PYRE_HIP(ctx, hipMalloc(&a->qmem, bb + wb)); PYRE_HIP(ctx, hipMalloc((void**)&a->qparams, 2 * (size_t)idx_hd * 4));
  PYRE_HIP(ctx, hipMemcpy(a->qparams, iqn_host, (size_t)idx_hd * 4, hipMemcpyHostToDevice)); PYRE_HIP(ctx, hipMemcpy(a->qparams + idx_hd, ikn_host, (size_t)idx_hd * 4, hipMemcpyHostToDevice));
  (void)hipFree(a->io); a->io = nullptr; PYRE_HIP(ctx, hipMalloc((void**)&a->io, 8 * (qw + (size_t)a->dv.nh * a->dv.hd) * 4));
  q.iqn = a->qparams; q.ikn = a->qparams + idx_hd; a->q = q;
  pyre_qsa_buf_carve(q, a->cap, a->qmem, &a->qb); pyre_qsa_work_carve(q, a->cap, (uint8_t*)a->qmem + bb, &a->qw);
  return PYRE_OK;
}
// Rebuilds the rotation table for a model context of ctx_tokens with a trained context of ctx_train (YaRN past it).
int pyre_attn_set_context(pyre_ctx* ctx, pyre_attn* a, int ctx_train, int ctx_tokens) {
  if (!ctx || !a) return pyre_fail(ctx, PYRE_E_ARG, "pyre_attn_set_context: null argument");
  if (a->len != 0) return pyre_fail(ctx, PYRE_E_STATE, "pyre_attn_set_context: the block already holds positions");
  std::vector<float> inv(a->dv.n_rot / 2 + 1); a->dv.mscale = pyre_rope_table(a->dv.n_rot, a->rope_base, ctx_train, ctx_tokens, inv.data());
  PYRE_HIP(ctx, hipMemcpy(a->params + 2 * a->dv.hd, inv.data(), (size_t)(a->dv.n_rot / 2) * 4, hipMemcpyHostToDevice)); return PYRE_OK;
}
// Harness access to the indexer: install the raw index keys of the a->len cached positions (their complete blocks are
// pooled on the device), read keys and pooled block keys back, read the positions the last call selected for token ti
// (*count = -1: dense).
int pyre_attn_load_index(pyre_ctx* ctx, pyre_attn* a, const float* ik_host) {
  if (!ctx || !a || !ik_host || a->q.nh < 1) return pyre_fail(ctx, PYRE_E_ARG, "pyre_attn_load_index: bad argument");
  if (a->len > 0) PYRE_HIP(ctx, hipMemcpyAsync(a->qb.ik, ik_host, (size_t)a->len * a->q.hd * 4, hipMemcpyHostToDevice, ctx->stream));
  int rc = pyre_qsa_pool_all(ctx, a->q, a->dv, a->qb, a->len); if (rc) return rc;
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}
int pyre_attn_read_index(pyre_ctx* ctx, pyre_attn* a, float* ik_host, float* ib_host) {
  if (!ctx || !a || a->q.nh < 1) return pyre_fail(ctx, PYRE_E_ARG, "pyre_attn_read_index: bad argument");
  const size_t hd = a->q.hd, nblk = (size_t)a->len / a->q.ratio, grp = (nblk + 63) / 64;
  if (ik_host && a->len > 0) PYRE_HIP(ctx, hipMemcpyAsync(ik_host, a->qb.ik, (size_t)a->len * hd * 4, hipMemcpyDeviceToHost, ctx->stream));
  std::vector<float> tmp(grp * hd * 64);
  if (ib_host && nblk > 0) PYRE_HIP(ctx, hipMemcpyAsync(tmp.data(), a->qb.ib, tmp.size() * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
  if (ib_host) for (size_t b = 0; b < nblk; ++b) for (size_t i = 0; i < hd; ++i) ib_host[b * hd + i] = tmp[qsa_ib_at(b, i, hd)];
  return PYRE_OK;
}
int pyre_attn_read_selection(pyre_ctx* ctx, pyre_attn* a, int ti, int32_t* pos_host, int cap, int32_t* count) {
  if (!ctx || !a || !count || a->q.nh < 1 || ti < 0 || ti >= 8) return pyre_fail(ctx, PYRE_E_ARG, "pyre_attn_read_selection: bad argument");
  PYRE_HIP(ctx, hipMemcpy(count, a->qw.pcount + ti, 4, hipMemcpyDeviceToHost));
  if (*count > 0 && pos_host) { int nrd = *count < cap ? *count : cap; PYRE_HIP(ctx, hipMemcpy(pos_host, a->qw.plist + (size_t)ti * a->qw.list_stride, (size_t)nrd * 4, hipMemcpyDeviceToHost)); }
  return PYRE_OK;
}
}  // extern "C"
