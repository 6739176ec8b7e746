// Decode attention (one query token) over an f16 KV cache with grouped-query heads.
//
// Split-K over the context: grid = (kv head, split).  A workgroup walks its slice of keys in
// tiles of 64 and serves all G = H/Hkv query heads of ONE kv head from a single pass over its
// K and V rows, so K/V are read from HBM once per kv head rather than once per query head.
// Scores and softmax statistics are fp32; each split keeps an online-softmax state (m, l, o)
// per query head and a second tiny kernel merges the splits with the usual log-sum-exp
// rescale.  (Merging inside the split kernel, by the last workgroup to arrive per kv head, was
// measured slower: store acknowledgement, arrival atomic and two rounds of agent-scope loads
// are four dependent memory round trips, more than the kernel boundary costs.)
//
// The decode step's own q/k/v can be taken raw from the stacked projection (QKV variant): the
// per-head RMSNorm and the rotary embedding of the query heads are redone in the prologue of
// every workgroup (a few hundred elements), and the workgroup whose chunk holds the new
// position also norms and rotates the new key, narrows key and value to f16, appends them to
// the cache and uses them straight from registers.  That removes the split-QKV/norm/RoPE/
// KV-write kernel (one launch, ~4.5 us per layer) from the decode step.
#include <algorithm>
#include <cstdlib>
#include <type_traits>
#include <cfloat>

#include "attention_keys.h"
#include "dh_common.h"

namespace {

constexpr int kTileKeys = dh::kAttnTileKeys;
constexpr int kMaxG = 8;       // query heads per kv head

using dh::DynKeys;
using dh::KeyRange;
using dh::splits_for;
using dh::max_splits_upto;
using dh::dyn_key_range;

struct AttnArgs {
  const float* Q;       // [H][D]
  const __half* K;      // [rows][Hkv][D]
  const __half* V;
  float* O;             // [H][D]
  float* ws;            // [H][nsplit of the launch][D + 2]  (o..., m, l)
  int H, Hkv, G, kbeg, kend, nsplit, tiles_per_split;
  int direct;           // one split and no merge launch behind it: the split kernel writes O itself
  float scale, softcap;
  int kv_start, ring_window;  // ring_window > 0: row = (kv_start + k) % ring_window
  // ---- QKV variant only
  const float* qkv;     // [(H + 2 Hkv) * D]: raw q heads, k heads, v heads of the step's token
  const float* qw;      // per-head RMSNorm weights [D] (null when use_norm == 0)
  const float* kw;
  const float* cos_row; // rotary tables at the row of this position: [rotary_dim / 2]
  const float* sin_row;
  __half* Kw;           // the caches again, writable
  __half* Vw;
  int64_t new_row;      // first element of the appended row in the caches
  int rotary_half, interleaved, w_offset, use_norm;
  float eps;
  int c_new, j_new;     // chunk, and key within the chunk, of the appended position
  // ---- key count on the device (dh_attn_decode_kvlen, dh_attn_decode_qkv_kvlen): kbeg, kend, nsplit,
  // direct and, for the stacked-projection form, cos_row, sin_row, new_row, c_new, j_new above are
  // derived in the kernel from the word behind kv_len_ptr; the grid holds the splits of max_kv_len
  DynKeys dyn;
  const float* cos_base;
  const float* sin_base;
};

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

typedef __attribute__((ext_vector_type(8))) _Float16 half8_t;

// Eight query values as one matrix-core operand: even operand rows take the f16 high parts of sc * q,
// odd rows what the high parts left over, so that the two rows together carry q to ~22 bits.  Both
// parts are rounded toward zero, two elements per instruction (the residual is exact in f32, so the
// rounding mode of the high part does not matter).  sc = 0 gives a zero operand.
__device__ __forceinline__ half8_t q_operand(const float (&qv)[8], const float sc, const bool odd) {
  typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
  u32x4 w;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const float x0 = qv[2 * i] * sc, x1 = qv[2 * i + 1] * sc;
    const uint32_t hi = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x0, x1));
    const float h0 = __half2float(__ushort_as_half((unsigned short)(hi & 0xffffu)));
    const float h1 = __half2float(__ushort_as_half((unsigned short)(hi >> 16)));
    const uint32_t lo = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x0 - h0, x1 - h1));
    w[i] = odd ? lo : hi;
  }
  return __builtin_bit_cast(half8_t, w);
}
typedef __attribute__((ext_vector_type(4))) float float4_t;


// Reductions across the lanes of a 16-lane row with DPP row shifts (no LDS traffic): afterwards
// the last lane of every aligned group of `span` lanes (span = 2, 4, 8 or 16) holds the
// group's result.
template <int CTRL>
__device__ __forceinline__ float dpp_row(float old, float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(v), CTRL, 0xF, 0xF, false));
}
template <int SPAN>
__device__ __forceinline__ float row_group_max(float v) {
  if (SPAN > 1) v = fmaxf(v, dpp_row<0x111>(v, v));
  if (SPAN > 2) v = fmaxf(v, dpp_row<0x112>(v, v));
  if (SPAN > 4) v = fmaxf(v, dpp_row<0x114>(v, v));
  if (SPAN > 8) v = fmaxf(v, dpp_row<0x118>(v, v));
  return v;
}
template <int SPAN>
__device__ __forceinline__ float row_group_sum(float v) {
  if (SPAN > 1) v += dpp_row<0x111>(0.f, v);
  if (SPAN > 2) v += dpp_row<0x112>(0.f, v);
  if (SPAN > 4) v += dpp_row<0x114>(0.f, v);
  if (SPAN > 8) v += dpp_row<0x118>(0.f, v);
  return v;
}

// One workgroup = one chunk of 64 keys of one kv head (or several chunks, strided, for long
// contexts), four waves, two barriers per chunk.
//   scores   wave w takes keys 16w..16w+15: S = Q.K^T with v_mfma_f32_16x16x32_f16.  The A
//            operand holds the G query heads of the kv head as rows (2g, 2g+1) = f16 high part
//            and f16 residual of scale*q (so q keeps ~22 bits); the B operand is loaded from
//            HBM directly in operand layout (lane (key, kg) reads 16 bytes of its key's row).
//   softmax  every wave redoes the (tiny) online-softmax update for all heads from the scores
//            in LDS, so no second exchange is needed: 64/GT lanes per head, GT keys per lane,
//            DPP row reductions, the per-head maxima and sums travel through scalar registers.
//   P.V      wave w owns output dims [D/4*w, D/4*(w+1)); lane (dq, kh) holds 4 dims of keys
//            kh, kh+KH, ... in registers and accumulates them for all heads; the key groups
//            meet in a wave-private LDS buffer at the end.
// K and V of the next chunk are requested before the current one is consumed.
// (Keeping two chunks in flight instead of one changed nothing, 34.1 vs 33.3 us at 32768 keys, and
// neither did 128-key chunks, 33.5 us: a workgroup's ~2 us per 64 keys is its own softmax and
// P.V arithmetic plus LDS round trips with one wave per SIMD, not the wait for memory or the
// barriers.)
// GT: query heads per kv head rounded up to 1, 2, 4 or 8 (bounds the unrolled per-head code).
// QKV: the step's q, k, v arrive raw (see the top of the file); the appended key is the last
// visible one, so the lanes that would read its row, or a clamped copy of it, from the not yet
// written cache are patched from registers.
template <int D, int GT, bool QKV>
__global__ __launch_bounds__(256) void attn_decode_split_kernel(const AttnArgs a_in) {
  AttnArgs a = a_in;
  // splits per query head in the workspace: the launch's split count, which with the key count on the
  // device is the largest any count can ask for, so that a reader finds a head's partial results
  // without knowing the count
  const int ws_stride = a.nsplit;
  if (a.dyn.kv_len_ptr != nullptr) {
    // the key count lives on the device: redo the host's arithmetic for it; surplus workgroups leave
    const KeyRange r = dyn_key_range(a.dyn);
    if ((int)blockIdx.y >= r.nsplit) return;
    a.kbeg = r.kbeg; a.kend = r.kend; a.nsplit = r.nsplit; a.direct = 0;
    if (QKV) {
      a.cos_row = a.cos_base + (int64_t)r.start_pos * a.rotary_half;
      a.sin_row = a.sin_base + (int64_t)r.start_pos * a.rotary_half;
      const int row = a.ring_window > 0 ? r.start_pos % a.ring_window : r.start_pos;
      a.new_row = (int64_t)row * a.Hkv * D;
      a.c_new = (r.kend - r.kbeg - 1) / kTileKeys;
      a.j_new = (r.kend - r.kbeg - 1) % kTileKeys;
    }
  }
  constexpr int STEPS = D / 32;          // MFMAs per 16 keys
  constexpr int DW = D / 4;              // output dims per wave
  constexpr int LPK = DW / 4;            // lanes per key in P.V (4 dims each)
  constexpr int KH = 64 / LPK;           // key groups
  constexpr int NJ = kTileKeys / KH;     // keys per lane
  constexpr int LH = 64 / GT;            // softmax: lanes per head (each holds GT keys)
  constexpr int SPAN = LH < 16 ? LH : 16;
  __shared__ __align__(16) float s_lds[GT][kTileKeys];        // raw scores of the chunk
  __shared__ __align__(16) float p_lds[4][GT][kTileKeys];     // per-wave probabilities
  __shared__ __align__(16) float o_lds[4][KH][GT][DW];        // per-wave partial outputs

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int kvh = blockIdx.x, split = blockIdx.y;
  const int G = a.G;
  const int64_t row_stride = (int64_t)a.Hkv * D;   // halves between consecutive keys
  const int qrow = lane & 15, kg = lane >> 4;
  const int dq = lane % LPK, kh = lane / LPK;
  const int key_s = 16 * wave + (lane & 15);
  const int nkeys_total = a.kend - a.kbeg;
  const int nchunks = (nkeys_total + kTileKeys - 1) / kTileKeys;

  uint4 kf[STEPS];
  uint2 vf[NJ], vn[NJ];
  // Requests this wave's 16 keys of K (into kf) and its dim slice of V (into vn) of chunk c.
#define DH_ATTN_LOAD(c_)                                                                          \
  do {                                                                                            \
    const int kbase_ = a.kbeg + (c_) * kTileKeys;                                                 \
    const int nk_ = min(kTileKeys, a.kend - kbase_);                                              \
    /* first cache row of the chunk; in ring layout rows wrap at the window (a chunk never */     \
    /* spans more keys than the window holds, so one conditional subtraction is enough)    */     \
    int row0_ = a.kv_start + kbase_, wrap_ = 0x7fffffff;                                          \
    if (a.ring_window > 0) {                                                                      \
      row0_ = (int)((unsigned)row0_ % (unsigned)a.ring_window);                                   \
      wrap_ = a.ring_window;                                                                      \
    }                                                                                             \
    int row_ = row0_ + min(key_s, nk_ - 1);                                                       \
    row_ = row_ >= wrap_ ? row_ - wrap_ : row_;                                                   \
    const __half* kp_ = a.K + (int64_t)row_ * row_stride + (int64_t)kvh * D + 8 * kg;             \
    _Pragma("unroll") for (int s = 0; s < STEPS; s++)                                             \
      kf[s] = *reinterpret_cast<const uint4*>(kp_ + 32 * s);                                      \
    _Pragma("unroll") for (int j = 0; j < NJ; j++) {                                              \
      int r_ = row0_ + min(kh + KH * j, nk_ - 1);                                                 \
      r_ = r_ >= wrap_ ? r_ - wrap_ : r_;                                                         \
      vn[j] = *reinterpret_cast<const uint2*>(a.V + (int64_t)r_ * row_stride + (int64_t)kvh * D + \
                                              DW * wave + 4 * dq);                                \
    }                                                                                             \
  } while (0)

  // The appended key/value in fragment form (QKV variant, owner workgroup): lanes whose key, or
  // whose clamped stand-in for a key past the end, is the appended one take it from here.
  uint4 knew[STEPS] = {};
  uint2 vnew = make_uint2(0u, 0u);
#define DH_ATTN_PATCH(c_)                                                                         \
  do {                                                                                            \
    if (QKV && (c_) == a.c_new) {                                                                 \
      if (key_s >= a.j_new) {                                                                     \
        _Pragma("unroll") for (int s = 0; s < STEPS; s++) kf[s] = knew[s];                        \
      }                                                                                           \
      _Pragma("unroll") for (int j = 0; j < NJ; j++)                                              \
        if (kh + KH * j >= a.j_new) vn[j] = vnew;                                                 \
    }                                                                                             \
  } while (0)

  if (!QKV && split < nchunks) DH_ATTN_LOAD(split);

  // ---- query fragments (A operand): row = lane & 15 -> head row>>1, high part / residual
  half8_t qa[STEPS];
  if constexpr (QKV) {
    // The rows of the step (G query heads; where the appended position is met, also the new key
    // and value) are prepared once per workgroup, one row per half wave (32 lanes x D/32
    // consecutive elements, so the loads are coalesced and tiny), and handed to the fragment
    // layout through LDS.  Their loads go out before those of the first K/V chunk, so they
    // return first and the preparation runs under the latency of the cache reads.
    constexpr int EPL = D / 32;                       // elements per lane
    constexpr int ROUNDS = (GT + 2 + 7) / 8;          // 8 half waves per round
    __shared__ __align__(16) float q_rows[GT][D];
    __shared__ __align__(16) __half k_row[D];
    __shared__ __align__(16) __half v_row[D];
    const bool owner = split == a.c_new % a.nsplit;
    const int hl = lane & 31;
    const int rotary_dim = 2 * a.rotary_half;
    float rx[ROUNDS][EPL], rw[ROUNDS][EPL], rc[ROUNDS][EPL], rs[ROUNDS][EPL];
    int role[ROUNDS];                                  // 0 idle, 1 query head, 2 new key, 3 new value
#pragma unroll
    for (int r = 0; r < ROUNDS; r++) {
      const int slot = 8 * r + 2 * wave + (lane >> 5);
      role[r] = slot < G ? 1 : (owner && slot == G) ? 2 : (owner && slot == G + 1) ? 3 : 0;
      const int64_t row = role[r] == 1 ? kvh * G + slot : role[r] == 2 ? a.H + kvh : role[r] == 3 ? a.H + a.Hkv + kvh : 0;
      const float* src = a.qkv + row * D + EPL * hl;
      const float* wsrc = !a.use_norm ? nullptr : role[r] == 1 ? a.qw : role[r] == 2 ? a.kw : nullptr;
      typedef __attribute__((ext_vector_type(EPL))) float row_vec_t;
      const row_vec_t xv = *reinterpret_cast<const row_vec_t*>(src);
      const row_vec_t wv = *reinterpret_cast<const row_vec_t*>((wsrc ? wsrc : a.qkv) + EPL * hl);
#pragma unroll
      for (int i = 0; i < EPL; i++) {
        const int e = EPL * hl + i;
        const bool rotated = (role[r] == 1 || role[r] == 2) && e < rotary_dim;
        const int p = a.interleaved ? e >> 1 : e & (a.rotary_half - 1);
        rx[r][i] = xv[i];
        rw[r][i] = wsrc ? wv[i] : 1.0f;
        rc[r][i] = a.cos_row[rotated ? p : 0];
        rs[r][i] = a.sin_row[rotated ? p : 0];
      }
    }
    DH_ATTN_LOAD(split);        // never empty: there are no more splits than chunks
#pragma unroll
    for (int r = 0; r < ROUNDS; r++) {
      const int slot = 8 * r + 2 * wave + (lane >> 5);
      float y[EPL];
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < EPL; i++) ss = fmaf(rx[r][i], rx[r][i], ss);
#pragma unroll
      for (int off = 1; off < 32; off <<= 1) ss += __shfl_xor(ss, off, 64);
      const bool normed = a.use_norm && (role[r] == 1 || role[r] == 2);
      const float inv = normed ? 1.0f / sqrtf(ss / (float)D + a.eps) : 1.0f;
#pragma unroll
      for (int i = 0; i < EPL; i++)
        y[i] = normed ? rx[r][i] * inv * (a.w_offset ? 1.0f + rw[r][i] : rw[r][i]) : rx[r][i];
      const bool rotates = role[r] == 1 || role[r] == 2;
      if (a.interleaved) {
#pragma unroll
        for (int i = 0; i < EPL; i += 2) {
          const float x0 = y[i], x1 = y[i + 1];
          const bool on = rotates && EPL * hl + i < rotary_dim;
          y[i] = on ? x0 * rc[r][i] - x1 * rs[r][i] : x0;
          y[i + 1] = on ? x0 * rs[r][i + 1] + x1 * rc[r][i + 1] : x1;
        }
      } else {
        const int pd = a.rotary_half / EPL;           // lanes between the partners (p, p + half)
        const bool low = EPL * hl < a.rotary_half;
#pragma unroll
        for (int i = 0; i < EPL; i++) {
          const float other = __shfl_xor(y[i], pd, 64);
          const float x0 = low ? y[i] : other, x1 = low ? other : y[i];
          const float rot = low ? x0 * rc[r][i] - x1 * rs[r][i] : x0 * rs[r][i] + x1 * rc[r][i];
          y[i] = rotates && EPL * hl + i < rotary_dim ? rot : y[i];
        }
      }
      if (role[r] == 1) {
#pragma unroll
        for (int i = 0; i < EPL; i++) q_rows[min(slot, GT - 1)][EPL * hl + i] = y[i];
      } else if (role[r] == 2 || role[r] == 3) {
        __half* lrow = role[r] == 2 ? k_row : v_row;
        __half* grow = (role[r] == 2 ? a.Kw : a.Vw) + a.new_row + (int64_t)kvh * D;
#pragma unroll
        for (int i = 0; i < EPL; i += 2) {
          const __half2 h2 = __floats2half2_rn(y[i], y[i + 1]);
          *reinterpret_cast<__half2*>(lrow + EPL * hl + i) = h2;
          *reinterpret_cast<__half2*>(grow + EPL * hl + i) = h2;
        }
      }
    }
    __syncthreads();
    const bool live = (qrow >> 1) < G;
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
      const float* qp = &q_rows[min(qrow >> 1, GT - 1)][32 * s + 8 * kg];
      const float4 q0 = reinterpret_cast<const float4*>(qp)[0], q1 = reinterpret_cast<const float4*>(qp)[1];
      const float qv[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
      qa[s] = q_operand(qv, live ? a.scale : 0.f, (qrow & 1) != 0);
    }
    if (owner) {
#pragma unroll
      for (int s = 0; s < STEPS; s++) knew[s] = *reinterpret_cast<const uint4*>(k_row + 32 * s + 8 * kg);
      vnew = *reinterpret_cast<const uint2*>(v_row + DW * wave + 4 * dq);
      DH_ATTN_PATCH(split);
    }
  } else {
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
#pragma unroll
      for (int i = 0; i < 8; i++) qa[s][i] = (_Float16)0.f;
      if ((qrow >> 1) < G) {
        const float* qp = a.Q + (int64_t)(kvh * G + (qrow >> 1)) * D + 32 * s + 8 * kg;
        const float4 q0 = reinterpret_cast<const float4*>(qp)[0], q1 = reinterpret_cast<const float4*>(qp)[1];
        const float qv[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        qa[s] = q_operand(qv, a.scale, (qrow & 1) != 0);
      }
    }
  }
  float m_run[GT], l_run[GT], acc[GT][4];
#pragma unroll
  for (int g = 0; g < GT; g++) {
    m_run[g] = -FLT_MAX; l_run[g] = 0.f;
    acc[g][0] = acc[g][1] = acc[g][2] = acc[g][3] = 0.f;
  }
  const int sm_g = lane / LH, sm_q = lane % LH;      // softmax role: head, key group

  for (int c = split; c < nchunks; c += a.nsplit) {
    const int kbase = a.kbeg + c * kTileKeys;
    const int nk = min(kTileKeys, a.kend - kbase);
    // ---- scores of 16 keys x G heads
    float4_t d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < STEPS; s++)
      d = __builtin_amdgcn_mfma_f32_16x16x32_f16(qa[s], __builtin_bit_cast(half8_t, kf[s]), d, 0, 0, 0);
#pragma unroll
    for (int j = 0; j < NJ; j++) vf[j] = vn[j];
    if (c + a.nsplit < nchunks) {
      DH_ATTN_LOAD(c + a.nsplit);
      DH_ATTN_PATCH(c + a.nsplit);
    }
    // lane (key, kg) holds rows 4kg..4kg+3 = heads 2kg (high + residual), 2kg+1
    {
      float sc2[2] = {d[0] + d[1], d[2] + d[3]};
      if (a.softcap > 0.f) {
#pragma unroll 1
        for (int e = 0; e < 2; e++) sc2[e] = tanhf(sc2[e] / a.softcap) * a.softcap;
      }
      const bool valid = key_s < nk;
      if (2 * kg < GT) s_lds[2 * kg][key_s] = valid ? sc2[0] : -FLT_MAX;
      if (2 * kg + 1 < GT) s_lds[2 * kg + 1][key_s] = valid ? sc2[1] : -FLT_MAX;
    }
    __syncthreads();
    // ---- online softmax: lane (head sm_g, group sm_q) owns keys sm_q*GT .. sm_q*GT + GT - 1
    {
      float sc[GT], pr[GT];
#pragma unroll
      for (int i = 0; i < GT; i++) sc[i] = s_lds[sm_g][sm_q * GT + i];
      float mx = sc[0];
#pragma unroll
      for (int i = 1; i < GT; i++) mx = fmaxf(mx, sc[i]);
      mx = row_group_max<SPAN>(mx);
      float m_new[GT], alpha[GT], my_m = 0.f;
#pragma unroll
      for (int g = 0; g < GT; g++) {
        float m = m_run[g];
#pragma unroll
        for (int r = 0; r < LH / SPAN; r++)       // the head's rows (or its single group)
          m = fmaxf(m, __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mx), g * LH + r * SPAN + SPAN - 1)));
        m_new[g] = m;
        alpha[g] = __expf(m_run[g] - m);
        if (g == sm_g) my_m = m;
      }
      float ps = 0.f;
#pragma unroll
      for (int i = 0; i < GT; i++) {
        pr[i] = sm_q * GT + i < nk ? __expf(sc[i] - my_m) : 0.f;
        ps += pr[i];
        p_lds[wave][sm_g][sm_q * GT + i] = pr[i];
      }
      ps = row_group_sum<SPAN>(ps);
#pragma unroll
      for (int g = 0; g < GT; g++) {
        float t = 0.f;
#pragma unroll
        for (int r = 0; r < LH / SPAN; r++)
          t += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ps), g * LH + r * SPAN + SPAN - 1));
        l_run[g] = l_run[g] * alpha[g] + t;
        m_run[g] = m_new[g];
        acc[g][0] *= alpha[g]; acc[g][1] *= alpha[g]; acc[g][2] *= alpha[g]; acc[g][3] *= alpha[g];
      }
    }
    // ---- P.V for this wave's dims (p_lds[wave] is private to the wave: program order suffices)
#pragma unroll
    for (int j = 0; j < NJ; j++) {
      const int key = kh + KH * j;
      const __half2* h2 = reinterpret_cast<const __half2*>(&vf[j]);
      const float2 v01 = __half22float2(h2[0]), v23 = __half22float2(h2[1]);
#pragma unroll
      for (int g = 0; g < GT; g++) {
        const float p = p_lds[wave][g][key];
        acc[g][0] = fmaf(p, v01.x, acc[g][0]);
        acc[g][1] = fmaf(p, v01.y, acc[g][1]);
        acc[g][2] = fmaf(p, v23.x, acc[g][2]);
        acc[g][3] = fmaf(p, v23.y, acc[g][3]);
      }
    }
    __syncthreads();     // s_lds is rewritten by the next chunk
  }
#undef DH_ATTN_LOAD
#undef DH_ATTN_PATCH

  // ---- key groups meet in the wave's LDS buffer, then the split's (o, m, l) go out
#pragma unroll
  for (int g = 0; g < GT; g++)
    *reinterpret_cast<float4*>(&o_lds[wave][kh][g][4 * dq]) = make_float4(acc[g][0], acc[g][1], acc[g][2], acc[g][3]);
#pragma unroll
  for (int t = 0; t < (GT * DW + 63) / 64; t++) {
    const int o = lane + 64 * t, g = min(o / DW, GT - 1), dim = o % DW;
    float v = 0.f;
#pragma unroll
    for (int k = 0; k < KH; k++) v += o_lds[wave][k][g][dim];
    if (o < GT * DW && g < G) {
      const int h = kvh * G + g;
      if (a.direct) {
        float l = 0.f;
#pragma unroll
        for (int gg = 0; gg < GT; gg++) l = gg == g ? l_run[gg] : l;
        a.O[(int64_t)h * D + DW * wave + dim] = l > 0.f ? v / l : 0.f;
      } else {
        a.ws[((int64_t)h * ws_stride + split) * (D + 2) + DW * wave + dim] = v;
      }
    }
  }
  if (!a.direct && wave == 0 && lane < G) {
    float* w = a.ws + ((int64_t)(kvh * G + lane) * ws_stride + split) * (D + 2);
    float mv = 0.f, lv = 0.f;
#pragma unroll
    for (int g = 0; g < GT; g++) {     // pick this lane's head without dynamic register indexing
      if (g == lane) { mv = m_run[g]; lv = l_run[g]; }
    }
    w[D] = mv;
    w[D + 1] = lv;
  }
}

// One workgroup per query head: out[d] = sum_s e^{m_s - M} o_s[d] / sum_s e^{m_s - M} l_s.
// Every load the kernel needs for the first 32 splits (a thread's 32 partial outputs, and one
// (m, l) pair per thread) is issued before anything is waited for, so the kernel costs one memory
// round trip, not one per dependent phase; splits beyond 32 follow in a pipelined loop.
// (Preloading 64 made short contexts slower, 8.9 vs 8.1 us at 512 keys.)
template <int D>
__global__ __launch_bounds__(D) void attn_decode_merge_kernel(const float* __restrict__ ws,
                                                              float* __restrict__ O, int nsplit, const DynKeys dyn) {
  constexpr int CH = 32;
  __shared__ float f_s[1024];
  __shared__ float red[4];
  const int h = blockIdx.x, d = threadIdx.x;
  const int ws_stride = nsplit;      // splits per head in the workspace (see the split kernel)
  if (dyn.kv_len_ptr != nullptr) {
    nsplit = dyn_key_range(dyn).nsplit;
    if (nsplit == 0) {            // no visible key: the output is zero, as the host path writes it
      O[(int64_t)h * D + d] = 0.f;
      return;
    }
  }
  const float* base = ws + (int64_t)h * ws_stride * (D + 2);
  float ov[CH];
#pragma unroll
  for (int i = 0; i < CH; i++) ov[i] = base[(int64_t)min(i, nsplit - 1) * (D + 2) + d];
  // (m, l) of split d, d + D, ...: registers for the first, reloaded (cache hits) beyond
  const bool has = d < nsplit;
  const float m0 = has ? base[d * (D + 2) + D] : -FLT_MAX;
  const float l0 = has ? base[d * (D + 2) + D + 1] : 0.f;
  float M = m0;
  for (int s = d + D; s < nsplit; s += D) M = fmaxf(M, base[s * (D + 2) + D]);
  M = wave_max(M);
  if ((d & 63) == 0) red[d >> 6] = M;
  __syncthreads();
  M = red[0];
  for (int w = 1; w < D / 64; w++) M = fmaxf(M, red[w]);
  __syncthreads();
  float den = 0.f;
  if (has) {
    const float f = __expf(m0 - M);
    f_s[d] = f;
    den = f * l0;
  }
  for (int s = d + D; s < nsplit; s += D) {
    const float f = __expf(base[s * (D + 2) + D] - M);
    f_s[s] = f;
    den = fmaf(f, base[s * (D + 2) + D + 1], den);
  }
  den = wave_sum(den);
  if ((d & 63) == 0) red[d >> 6] = den;
  __syncthreads();
  den = 0.f;
  for (int w = 0; w < D / 64; w++) den += red[w];
  float num = 0.f;
#pragma unroll
  for (int i = 0; i < CH; i++) num = i < nsplit ? fmaf(f_s[i], ov[i], num) : num;
#pragma unroll 8
  for (int s = CH; s < nsplit; s++) num = fmaf(f_s[s], base[s * (D + 2) + d], num);
  O[(int64_t)h * D + d] = den > 0.f ? num / den : 0.f;
}

__global__ void zero_f32_kernel(float* p, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

int max_splits_for(int kv_len) { return std::max(1, (kv_len + kTileKeys - 1) / kTileKeys); }

int one_per_cu_for(int Hkv) { return dh::attn_one_per_cu(dh::num_cus(), Hkv); }

int choose_splits(int Hkv, int nkeys) {
  const int tiles = std::max(1, (nkeys + kTileKeys - 1) / kTileKeys);
  static const double env_per_cu = dh::tuning_double("DH_ATTN_WG_PER_CU", 0.0);
  const int one_per_cu = one_per_cu_for(Hkv);
  if (env_per_cu > 0.0) return std::min(tiles, std::max(1, (int)(one_per_cu * env_per_cu)));
  return splits_for(one_per_cu, nkeys);
}

typedef void (*SplitKernel)(const AttnArgs);
typedef void (*MergeKernel)(const float*, float*, int, const DynKeys);

template <int D, bool QKV>
SplitKernel split_kernel_for(int G) {
  if (G <= 1) return attn_decode_split_kernel<D, 1, QKV>;
  if (G <= 2) return attn_decode_split_kernel<D, 2, QKV>;
  if (G <= 4) return attn_decode_split_kernel<D, 4, QKV>;
  return attn_decode_split_kernel<D, 8, QKV>;
}
SplitKernel split_kernel_for(int D, bool qkv, int G) {
  if (D == 64) return qkv ? split_kernel_for<64, true>(G) : split_kernel_for<64, false>(G);
  return qkv ? split_kernel_for<128, true>(G) : split_kernel_for<128, false>(G);
}
MergeKernel merge_kernel_for(int D) { return D == 64 ? attn_decode_merge_kernel<64> : attn_decode_merge_kernel<128>; }

int launch(const AttnArgs& a, int D, bool qkv, const char* op, bool merge = true) {
  hipLaunchKernelGGL(split_kernel_for(D, qkv, a.G), dim3(a.Hkv, a.nsplit), dim3(256), 0, dh::stream(), a);
  DH_CHECK_LAUNCH(op);
  if (!a.direct && merge) {
    hipLaunchKernelGGL(merge_kernel_for(D), dim3(a.H), dim3(D), 0, dh::stream(), a.ws, a.O, a.nsplit, a.dyn);
    DH_CHECK_LAUNCH(op);
  }
  return 0;
}

// Host-side arithmetic of one decode attention call at position shift `delta` from the recorded one:
// visible key range, key splits, and for the stacked-projection form the rotary rows and the
// appended cache row.  Returns 1 when no key is visible (the caller zero-fills O), 0 otherwise.
int build_args(const dh::GraphAttnCall& c, int delta, bool force_merge, AttnArgs& a) {
  const int start_pos = c.start_pos + delta;
  const int kv_len = c.kv_len + delta;
  int64_t kbeg = 0, kend;
  if (c.qkv) {
    kend = (int64_t)start_pos - c.kv_start + 1;
  } else {
    kend = kv_len;
    if (c.causal) kend = std::min<int64_t>(kend, (int64_t)start_pos - c.kv_start + 1);
  }
  if (c.sliding_window > 0 && start_pos >= c.sliding_window)
    kbeg = std::max<int64_t>(0, (int64_t)start_pos - c.sliding_window + 1 - c.kv_start);
  if (kend <= kbeg) return 1;
  a = AttnArgs{};
  a.K = static_cast<const __half*>(c.K); a.V = static_cast<const __half*>(c.V);
  a.O = c.O; a.ws = static_cast<float*>(c.ws);
  a.H = c.H; a.Hkv = c.Hkv; a.G = c.H / c.Hkv;
  a.kbeg = (int)kbeg; a.kend = (int)kend;
  const int nkeys = (int)(kend - kbeg);
  a.nsplit = choose_splits(c.Hkv, nkeys);
  a.direct = (a.nsplit == 1 && !force_merge) ? 1 : 0;
  a.scale = c.scale; a.softcap = c.softcap;
  a.kv_start = c.kv_start;
  a.ring_window = c.kv_layout == DH_KV_RING ? c.sliding_window : 0;
  if (c.qkv) {
    const int half = c.rotary_dim / 2;
    a.Kw = static_cast<__half*>(c.K); a.Vw = static_cast<__half*>(c.V);
    a.qkv = c.q; a.qw = c.qw; a.kw = c.kw;
    a.cos_row = c.cos + (int64_t)start_pos * half;
    a.sin_row = c.sin + (int64_t)start_pos * half;
    a.rotary_half = half; a.interleaved = c.interleaved; a.w_offset = c.weight_offset; a.use_norm = c.use_norm;
    a.eps = c.eps;
    const int64_t row = a.ring_window > 0 ? start_pos % a.ring_window : start_pos;
    a.new_row = row * c.Hkv * c.D;
    a.c_new = (nkeys - 1) / kTileKeys;
    a.j_new = (nkeys - 1) % kTileKeys;
  } else {
    a.Q = c.q;
  }
  return 0;
}

}  // namespace

// ---------------------------------------------------------------------------------------
// Split-K partials for callers that may not allocate (dh_attn_decode_static): a fixed array in
// device memory that belongs to the library.  Each GPU holds its own copy at its own address, so
// the address is asked for once per device (dh_init) and kept; host code only ever passes that
// address, never the symbol, to kernels.
// ---------------------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = (size_t)4 << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static void* g_scratch_ptr[kMaxDevices] = {};

namespace dh {
// The captured graph is a chain (one stream): walking it from its root visits the kernel nodes in
// launch order.  Every recorded attention call owns the next node that runs its split kernel and
// the merge node behind it.
int attn_graph_bind(Graph* g) {
  if (g->n_attn == 0) return 0;
  size_t n = 0;
  DH_CHECK_HIP("dh_graph_end", hipGraphGetNodes(g->graph, nullptr, &n));
  hipGraphNode_t* nodes = new hipGraphNode_t[n ? n : 1];
  hipError_t e = hipGraphGetNodes(g->graph, nodes, &n);
  if (e != hipSuccess) {
    delete[] nodes;
    return fail(2, "[dh_graph_end] hipGraphGetNodes failed: %s", hipGetErrorString(e));
  }
  // order the nodes along the chain: repeatedly take the node whose dependencies are all placed
  hipGraphNode_t* order = new hipGraphNode_t[n ? n : 1];
  size_t placed = 0;
  {
    size_t nroot = 0;
    e = hipGraphGetRootNodes(g->graph, nullptr, &nroot);
    hipGraphNode_t cur = nullptr;
    if (e == hipSuccess && nroot == 1) e = hipGraphGetRootNodes(g->graph, &cur, &nroot);
    if (e != hipSuccess || nroot != 1) {
      delete[] nodes; delete[] order;
      return fail(2, "[dh_graph_end] the captured graph is not a single chain (%zu roots)", nroot);
    }
    while (cur && placed < n) {
      order[placed++] = cur;
      size_t nd = 0;
      if (hipGraphNodeGetDependentNodes(cur, nullptr, &nd) != hipSuccess || nd > 1) {
        delete[] nodes; delete[] order;
        return fail(2, "[dh_graph_end] the captured graph is not a single chain");
      }
      hipGraphNode_t next = nullptr;
      if (nd == 1 && hipGraphNodeGetDependentNodes(cur, &next, &nd) != hipSuccess) next = nullptr;
      cur = nd == 1 ? next : nullptr;
    }
  }
  delete[] nodes;
  int ci = 0;
  bool want_merge = false;
  for (size_t i = 0; i < placed && ci <= g->n_attn; i++) {
    hipGraphNodeType type;
    if (hipGraphNodeGetType(order[i], &type) != hipSuccess || type != hipGraphNodeTypeKernel) continue;
    hipKernelNodeParams kp{};
    if (hipGraphKernelNodeGetParams(order[i], &kp) != hipSuccess) continue;
    if (want_merge) {
      if (kp.func == reinterpret_cast<void*>(merge_kernel_for(g->attn[ci].D))) {
        g->attn[ci].merge_node = order[i];
        want_merge = false;
        ci++;
      }
      continue;
    }
    if (ci < g->n_attn) {
      const GraphAttnCall& c = g->attn[ci];
      if (kp.func == reinterpret_cast<void*>(split_kernel_for(c.D, c.qkv != 0, c.H / c.Hkv))) {
        g->attn[ci].split_node = order[i];
        want_merge = true;
      }
    }
  }
  delete[] order;
  if (ci != g->n_attn || want_merge)
    return fail(2, "[dh_graph_end] found the kernel nodes of %d of %d attention calls in the captured graph", ci, g->n_attn);
  return 0;
}

int attn_graph_set_position(Graph* g, int position) {
  const int delta = position - g->captured_position;
  for (int i = 0; i < g->n_attn; i++) {
    const GraphAttnCall& c = g->attn[i];
    AttnArgs a;
    if (build_args(c, delta, true, a))
      return fail(1, "[dh_graph_launch] position %d leaves attention call %d without a visible key", position, i);
    // the split partials of the new position must fit where the captured call put them
    const size_t ws_need = (size_t)c.H * a.nsplit * (c.D + 2) * sizeof(float);
    if (c.ws_capacity && ws_need > c.ws_capacity)
      return fail(1, "[dh_graph_launch] position %d needs %zu bytes of split partials in attention call %d, the library's "
                  "scratch holds %zu", position, ws_need, i, c.ws_capacity);
    AttnArgs* ap = &a;
    void* split_args[] = {ap};
    hipKernelNodeParams sp{};
    sp.func = reinterpret_cast<void*>(split_kernel_for(c.D, c.qkv != 0, a.G));
    sp.gridDim = dim3(a.Hkv, a.nsplit);
    sp.blockDim = dim3(256);
    sp.sharedMemBytes = 0;
    sp.kernelParams = split_args;
    DH_CHECK_HIP("dh_graph_launch", hipGraphExecKernelNodeSetParams(g->exec, c.split_node, &sp));
    const float* ws = a.ws;
    float* O = a.O;
    int nsplit = a.nsplit;
    DynKeys dyn = a.dyn;
    void* merge_args[] = {&ws, &O, &nsplit, &dyn};
    hipKernelNodeParams mp{};
    mp.func = reinterpret_cast<void*>(merge_kernel_for(c.D));
    mp.gridDim = dim3(a.H);
    mp.blockDim = dim3(c.D);
    mp.sharedMemBytes = 0;
    mp.kernelParams = merge_args;
    DH_CHECK_HIP("dh_graph_launch", hipGraphExecKernelNodeSetParams(g->exec, c.merge_node, &mp));
  }
  return 0;
}

int attn_static_scratch_init(int device) {
  if (device < 0 || device >= kMaxDevices)
    return fail(1, "[dh_init] device ordinal %d is beyond the %d the static attention scratch tracks", device, kMaxDevices);
  if (g_scratch_ptr[device]) return 0;
  void* ptr = nullptr;
  DH_CHECK_HIP("dh_init", hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
  g_scratch_ptr[device] = ptr;
  return 0;
}
}  // namespace dh


extern "C" {

size_t dh_attn_decode_workspace_bytes(int H, int D, int kv_len) {
  if (H <= 0 || D <= 0 || kv_len <= 0) return 256;
  const size_t splits = (size_t)std::min(max_splits_for(kv_len), 1024);
  return std::max<size_t>(256, (size_t)H * splits * (D + 2) * sizeof(float));
}

// Shared body of dh_attn_decode and dh_attn_decode_static.  ws_capacity: bytes behind d_workspace when
// the caller of this function knows them (0: the public contract, dh_attn_decode_workspace_bytes, holds).
static int attn_decode_impl(const char* op, const float* d_Q, const void* d_K, const void* d_V, float* d_O, int H,
                            int Hkv, int D, int kv_len, float scale, int causal, int start_pos, float softcap,
                            int sliding_window, int kv_start, int kv_layout, void* d_workspace, size_t ws_capacity) {
  DH_REQUIRE_INIT(op);
  if (H <= 0 || Hkv <= 0 || D <= 0) return dh::fail(1, "[%s] numHeads/numKVHeads/headDim must be positive", op);
  if (H % Hkv) return dh::fail(1, "[%s] numHeads=%d must be a multiple of numKVHeads=%d", op, H, Hkv);
  const int G = H / Hkv;
  if (G > kMaxG) return dh::fail(1, "[%s] %d query heads per kv head not supported (max %d)", op, G, kMaxG);
  if (D != 64 && D != 128) return dh::fail(1, "[%s] headDim %d not supported (64, 128)", op, D);
  if ((int64_t)G * D > 2048) return dh::fail(1, "[%s] G*headDim=%d exceeds 2048", op, G * D);
  if (kv_len < 0 || start_pos < 0 || sliding_window < 0 || kv_start < 0)
    return dh::fail(1, "[%s] kvLen, startPos, slidingWindow and kvStart must be non-negative", op);
  if (kv_layout != DH_KV_CONTIGUOUS && kv_layout != DH_KV_RING)
    return dh::fail(1, "[%s] kvLayout %d not supported (contiguous, ring)", op, kv_layout);
  if (kv_layout == DH_KV_RING && sliding_window <= 0)
    return dh::fail(1, "[%s] ring layout needs slidingWindow > 0", op);
  if (!d_Q || !d_O) return dh::fail(1, "[%s] null pointer", op);

  dh::GraphAttnCall c{};
  c.qkv = 0; c.q = d_Q; c.K = const_cast<void*>(d_K); c.V = const_cast<void*>(d_V); c.O = d_O;
  c.H = H; c.Hkv = Hkv; c.D = D; c.kv_len = kv_len; c.start_pos = start_pos; c.causal = causal;
  c.scale = scale; c.softcap = softcap; c.sliding_window = sliding_window; c.kv_start = kv_start;
  c.kv_layout = kv_layout; c.ws = d_workspace; c.ws_capacity = ws_capacity;
  const bool capturing = dh::capturing_graph() != nullptr;
  AttnArgs a;
  if (build_args(c, 0, capturing, a)) {
    if (capturing) return dh::fail(1, "[%s] a captured step needs at least one visible key", op);
    hipLaunchKernelGGL(zero_f32_kernel, dim3((H * D + 255) / 256), dim3(256), 0, dh::stream(), d_O, H * D);
    DH_CHECK_LAUNCH(op);
    return 0;
  }
  if (!d_K || !d_V) return dh::fail(1, "[%s] null pointer", op);
  if ((reinterpret_cast<uintptr_t>(d_K) | reinterpret_cast<uintptr_t>(d_V)) & 15)
    return dh::fail(1, "[%s] K/V pointers must be 16-byte aligned", op);
  if (!a.direct && !d_workspace) return dh::fail(1, "[%s] workspace is required", op);
  const size_t ws_need = a.direct ? 0 : (size_t)H * a.nsplit * (D + 2) * sizeof(float);
  if (ws_capacity && ws_need > ws_capacity)
    return dh::fail(1, "[%s] numHeads=%d, headDim=%d with %d key splits needs %zu bytes of split partials, the "
                       "scratch holds %zu: use dh_attn_decode with a workspace", op, H, D, a.nsplit, ws_need, ws_capacity);
  dh::graph_note_attention(c);
  return launch(a, D, false, op);
}

int dh_attn_decode(const float* d_Q, const void* d_K, const void* d_V, float* d_O, int H, int Hkv, int D,
                   int kv_len, float scale, int causal, int start_pos, float softcap, int sliding_window,
                   int kv_start, int kv_layout, void* d_workspace) {
  return attn_decode_impl("dh_attn_decode", d_Q, d_K, d_V, d_O, H, Hkv, D, kv_len, scale, causal, start_pos, softcap,
                          sliding_window, kv_start, kv_layout, d_workspace, 0);
}

size_t dh_attn_decode_static_max_bytes(void) { return kStaticScratchBytes; }

int dh_attn_decode_static(const float* d_Q, const void* d_K, const void* d_V, float* d_O, int H, int Hkv, int D,
                          int kv_len, float scale, int causal, int start_pos, float softcap, int sliding_window,
                          int kv_start, int kv_layout) {
  const char* op = "dh_attn_decode_static";
  DH_REQUIRE_INIT(op);
  int device = -1;
  DH_CHECK_HIP(op, hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices || !g_scratch_ptr[device])
    return dh::fail(1, "[%s] the static scratch of device %d was not set up by dh_init", op, device);
  // nothing in the scratch has to start at zero: every (head, split) slot the merge reads is
  // written by the split kernel of the same call
  return attn_decode_impl(op, d_Q, d_K, d_V, d_O, H, Hkv, D, kv_len, scale, causal, start_pos, softcap,
                          sliding_window, kv_start, kv_layout, g_scratch_ptr[device], kStaticScratchBytes);
}

int dh_attn_decode_qkv_supported(int H, int Hkv, int D, int rotary_dim, int interleaved) {
  if (H <= 0 || Hkv <= 0 || H % Hkv || H / Hkv > kMaxG || (D != 64 && D != 128)) return 0;
  if (rotary_dim <= 0 || rotary_dim > D || rotary_dim % 2) return 0;
  if (interleaved) return 1;                       // pairs (2p, 2p + 1): always inside one lane
  // pairs (p, p + half): half a power of two and at least one lane's D/32 elements
  return (rotary_dim & (rotary_dim - 1)) == 0 && rotary_dim / 2 >= D / 32;
}

// Shared body of dh_attn_decode_qkv and dh_attn_decode_qkv_partials (out_nsplit != null: the splits'
// partial results stay in the workspace, no merge launch, *out_nsplit receives their number).
static int attn_decode_qkv_impl(const char* op, const float* d_qkv, const float* d_q_weight, const float* d_k_weight,
                                const float* d_cos, const float* d_sin, void* d_cache_k, void* d_cache_v, float* d_O, int H,
                                int Hkv, int D, int start_pos, int rotary_dim, int interleaved, float eps, int weight_offset,
                                int use_norm, float scale, float softcap, int sliding_window, int kv_start, int kv_layout,
                                void* d_workspace, int* out_nsplit) {
  DH_REQUIRE_INIT(op);
  const bool partials = out_nsplit != nullptr;
  if (H <= 0 || Hkv <= 0 || D <= 0) return dh::fail(1, "[%s] numHeads/numKVHeads/headDim must be positive", op);
  if (H % Hkv) return dh::fail(1, "[%s] numHeads=%d must be a multiple of numKVHeads=%d", op, H, Hkv);
  if (!dh_attn_decode_qkv_supported(H, Hkv, D, rotary_dim, interleaved))
    return dh::fail(1, "[%s] shape not served (heads %d/%d, headDim %d, rotaryDim %d, interleaved %d): use "
                       "dh_qkv_norm_rope_kvwrite + dh_attn_decode", op, H, Hkv, D, rotary_dim, interleaved);
  if (start_pos < 0 || sliding_window < 0 || kv_start < 0 || kv_start > start_pos)
    return dh::fail(1, "[%s] need 0 <= kvStart <= startPos and slidingWindow >= 0", op);
  if (kv_layout != DH_KV_CONTIGUOUS && kv_layout != DH_KV_RING)
    return dh::fail(1, "[%s] kvLayout %d not supported (contiguous, ring)", op, kv_layout);
  if (kv_layout == DH_KV_RING && sliding_window <= 0)
    return dh::fail(1, "[%s] ring layout needs slidingWindow > 0", op);
  if (!d_qkv || !d_cos || !d_sin || !d_cache_k || !d_cache_v || (!d_O && !partials)) return dh::fail(1, "[%s] null pointer", op);
  if (use_norm && (!d_q_weight || !d_k_weight)) return dh::fail(1, "[%s] q/k norm weights are required", op);
  if ((reinterpret_cast<uintptr_t>(d_cache_k) | reinterpret_cast<uintptr_t>(d_cache_v) |
       reinterpret_cast<uintptr_t>(d_qkv) | reinterpret_cast<uintptr_t>(d_q_weight) |
       reinterpret_cast<uintptr_t>(d_k_weight)) & 15)
    return dh::fail(1, "[%s] qkv, the norm weights and the caches must be 16-byte aligned", op);
  dh::GraphAttnCall c{};
  c.qkv = 1; c.q = d_qkv; c.qw = d_q_weight; c.kw = d_k_weight; c.cos = d_cos; c.sin = d_sin;
  c.K = d_cache_k; c.V = d_cache_v; c.O = d_O;
  c.H = H; c.Hkv = Hkv; c.D = D; c.kv_len = start_pos - kv_start + 1; c.start_pos = start_pos; c.causal = 1;
  c.rotary_dim = rotary_dim; c.interleaved = interleaved; c.weight_offset = weight_offset; c.use_norm = use_norm;
  c.eps = eps; c.scale = scale; c.softcap = softcap; c.sliding_window = sliding_window; c.kv_start = kv_start;
  c.kv_layout = kv_layout; c.ws = d_workspace;
  const bool capturing = dh::capturing_graph() != nullptr;
  // (a consumer of the partial results is given the split count of THIS position: a replay at another
  // position would need both patched, so the captured form is the one with the key count on the device)
  if (partials && capturing)
    return dh::fail(1, "[%s] not while a graph is being captured: use dh_attn_decode_qkv_kvlen_partials there", op);
  AttnArgs a;
  if (build_args(c, 0, capturing || partials, a)) return dh::fail(2, "[%s] internal: no visible key", op);
  if (!a.direct && !d_workspace) return dh::fail(1, "[%s] workspace is required", op);
  if (partials) {
    *out_nsplit = a.nsplit;
    return launch(a, D, true, op, false);
  }
  dh::graph_note_attention(c);
  return launch(a, D, true, op);
}

int dh_attn_decode_qkv(const float* d_qkv, const float* d_q_weight, const float* d_k_weight, const float* d_cos,
                       const float* d_sin, void* d_cache_k, void* d_cache_v, float* d_O, int H, int Hkv, int D,
                       int start_pos, int rotary_dim, int interleaved, float eps, int weight_offset, int use_norm,
                       float scale, float softcap, int sliding_window, int kv_start, int kv_layout,
                       void* d_workspace) {
  return attn_decode_qkv_impl("dh_attn_decode_qkv", d_qkv, d_q_weight, d_k_weight, d_cos, d_sin, d_cache_k, d_cache_v, d_O, H,
                              Hkv, D, start_pos, rotary_dim, interleaved, eps, weight_offset, use_norm, scale, softcap,
                              sliding_window, kv_start, kv_layout, d_workspace, nullptr);
}

int dh_attn_decode_qkv_partials(const float* d_qkv, const float* d_q_weight, const float* d_k_weight, const float* d_cos,
                                const float* d_sin, void* d_cache_k, void* d_cache_v, int H, int Hkv, int D, int start_pos,
                                int rotary_dim, int interleaved, float eps, int weight_offset, int use_norm, float scale,
                                float softcap, int sliding_window, int kv_start, int kv_layout, void* d_workspace,
                                int* out_nsplit) {
  const char* op = "dh_attn_decode_qkv_partials";
  if (!out_nsplit) return dh::fail(1, "[%s] out_nsplit is null", op);
  return attn_decode_qkv_impl(op, d_qkv, d_q_weight, d_k_weight, d_cos, d_sin, d_cache_k, d_cache_v, nullptr, H, Hkv, D,
                              start_pos, rotary_dim, interleaved, eps, weight_offset, use_norm, scale, softcap,
                              sliding_window, kv_start, kv_layout, d_workspace, out_nsplit);
}

// ---- key count on the device -------------------------------------------------------------------
// Shared body of dh_attn_decode_kvlen and dh_attn_decode_qkv_kvlen: the launch arguments are built
// for max_kv_len keys (that fixes pointers, shapes and the grid), the kernels replace everything
// that depends on the key count by what the device word says.
static int attn_decode_kvlen_impl(const char* op, dh::GraphAttnCall c, const uint32_t* d_kv_len, int max_kv_len,
                                  int start_pos, bool merge = true) {
  if (!d_kv_len) return dh::fail(1, "[%s] the key-count pointer is null", op);
  if (reinterpret_cast<uintptr_t>(d_kv_len) & 3) return dh::fail(1, "[%s] the key-count pointer must be 4-byte aligned", op);
  if (max_kv_len < 1) return dh::fail(1, "[%s] max_kv_len must be at least 1", op);
  if (!c.ws) return dh::fail(1, "[%s] workspace is required", op);
  c.kv_len = max_kv_len;
  c.start_pos = start_pos < 0 ? c.kv_start + max_kv_len - 1 : start_pos;
  AttnArgs a;
  if (build_args(c, 0, true, a)) return dh::fail(1, "[%s] no key is visible even at max_kv_len=%d", op, max_kv_len);
  const int one_per_cu = one_per_cu_for(c.Hkv);
  a.dyn = DynKeys{d_kv_len, max_kv_len, c.causal, start_pos, c.sliding_window, c.kv_start, c.qkv, one_per_cu};
  a.cos_base = c.cos;
  a.sin_base = c.sin;
  a.nsplit = max_splits_upto(one_per_cu, max_kv_len);      // the grid; the kernels use the device word's split count
  a.direct = 0;
  // nothing is recorded for graph replays: a captured launch follows the device word by itself
  return launch(a, c.D, c.qkv != 0, op, merge);
}

int dh_attn_decode_kvlen(const float* d_Q, const void* d_K, const void* d_V, float* d_O, int H, int Hkv, int D,
                         const uint32_t* d_kv_len, int max_kv_len, float scale, int causal, int start_pos,
                         float softcap, int sliding_window, int kv_start, int kv_layout, void* d_workspace) {
  const char* op = "dh_attn_decode_kvlen";
  DH_REQUIRE_INIT(op);
  if (H <= 0 || Hkv <= 0 || D <= 0) return dh::fail(1, "[%s] numHeads/numKVHeads/headDim must be positive", op);
  if (H % Hkv) return dh::fail(1, "[%s] numHeads=%d must be a multiple of numKVHeads=%d", op, H, Hkv);
  const int G = H / Hkv;
  if (G > kMaxG) return dh::fail(1, "[%s] %d query heads per kv head not supported (max %d)", op, G, kMaxG);
  if (D != 64 && D != 128) return dh::fail(1, "[%s] headDim %d not supported (64, 128)", op, D);
  if (sliding_window < 0 || kv_start < 0) return dh::fail(1, "[%s] slidingWindow and kvStart must be non-negative", op);
  if (kv_layout != DH_KV_CONTIGUOUS && kv_layout != DH_KV_RING)
    return dh::fail(1, "[%s] kvLayout %d not supported (contiguous, ring)", op, kv_layout);
  if (kv_layout == DH_KV_RING && sliding_window <= 0) return dh::fail(1, "[%s] ring layout needs slidingWindow > 0", op);
  if (!d_Q || !d_O || !d_K || !d_V) return dh::fail(1, "[%s] null pointer", op);
  if ((reinterpret_cast<uintptr_t>(d_K) | reinterpret_cast<uintptr_t>(d_V)) & 15)
    return dh::fail(1, "[%s] K/V pointers must be 16-byte aligned", op);
  dh::GraphAttnCall c{};
  c.qkv = 0; c.q = d_Q; c.K = const_cast<void*>(d_K); c.V = const_cast<void*>(d_V); c.O = d_O;
  c.H = H; c.Hkv = Hkv; c.D = D; c.causal = causal;
  c.scale = scale; c.softcap = softcap; c.sliding_window = sliding_window; c.kv_start = kv_start;
  c.kv_layout = kv_layout; c.ws = d_workspace;
  return attn_decode_kvlen_impl(op, c, d_kv_len, max_kv_len, start_pos);
}

static int attn_decode_qkv_kvlen_impl(const char* op, bool partials, const float* d_qkv, const float* d_q_weight,
                                      const float* d_k_weight, const float* d_cos, const float* d_sin, void* d_cache_k,
                                      void* d_cache_v, float* d_O, int H, int Hkv, int D, const uint32_t* d_kv_len,
                                      int max_kv_len, int rotary_dim, int interleaved, float eps, int weight_offset,
                                      int use_norm, float scale, float softcap, int sliding_window, int kv_start,
                                      int kv_layout, void* d_workspace) {
  DH_REQUIRE_INIT(op);
  if (H <= 0 || Hkv <= 0 || D <= 0) return dh::fail(1, "[%s] numHeads/numKVHeads/headDim must be positive", op);
  if (H % Hkv) return dh::fail(1, "[%s] numHeads=%d must be a multiple of numKVHeads=%d", op, H, Hkv);
  if (!dh_attn_decode_qkv_supported(H, Hkv, D, rotary_dim, interleaved))
    return dh::fail(1, "[%s] shape not served (heads %d/%d, headDim %d, rotaryDim %d, interleaved %d): use "
                       "dh_qkv_norm_rope_kvwrite + dh_attn_decode_kvlen", op, H, Hkv, D, rotary_dim, interleaved);
  if (sliding_window < 0 || kv_start < 0) return dh::fail(1, "[%s] slidingWindow and kvStart must be non-negative", op);
  if (kv_layout != DH_KV_CONTIGUOUS && kv_layout != DH_KV_RING)
    return dh::fail(1, "[%s] kvLayout %d not supported (contiguous, ring)", op, kv_layout);
  if (kv_layout == DH_KV_RING && sliding_window <= 0) return dh::fail(1, "[%s] ring layout needs slidingWindow > 0", op);
  if (!d_qkv || !d_cos || !d_sin || !d_cache_k || !d_cache_v || (!d_O && !partials)) return dh::fail(1, "[%s] null pointer", op);
  if (use_norm && (!d_q_weight || !d_k_weight)) return dh::fail(1, "[%s] q/k norm weights are required", op);
  if ((reinterpret_cast<uintptr_t>(d_cache_k) | reinterpret_cast<uintptr_t>(d_cache_v) |
       reinterpret_cast<uintptr_t>(d_qkv) | reinterpret_cast<uintptr_t>(d_q_weight) |
       reinterpret_cast<uintptr_t>(d_k_weight)) & 15)
    return dh::fail(1, "[%s] qkv, the norm weights and the caches must be 16-byte aligned", op);
  dh::GraphAttnCall c{};
  c.qkv = 1; c.q = d_qkv; c.qw = d_q_weight; c.kw = d_k_weight; c.cos = d_cos; c.sin = d_sin;
  c.K = d_cache_k; c.V = d_cache_v; c.O = d_O;
  c.H = H; c.Hkv = Hkv; c.D = D; c.causal = 1;
  c.rotary_dim = rotary_dim; c.interleaved = interleaved; c.weight_offset = weight_offset; c.use_norm = use_norm;
  c.eps = eps; c.scale = scale; c.softcap = softcap; c.sliding_window = sliding_window; c.kv_start = kv_start;
  c.kv_layout = kv_layout; c.ws = d_workspace;
  return attn_decode_kvlen_impl(op, c, d_kv_len, max_kv_len, -1, !partials);
}

int dh_attn_decode_qkv_kvlen(const float* d_qkv, const float* d_q_weight, const float* d_k_weight, const float* d_cos,
                             const float* d_sin, void* d_cache_k, void* d_cache_v, float* d_O, int H, int Hkv, int D,
                             const uint32_t* d_kv_len, int max_kv_len, int rotary_dim, int interleaved, float eps,
                             int weight_offset, int use_norm, float scale, float softcap, int sliding_window,
                             int kv_start, int kv_layout, void* d_workspace) {
  return attn_decode_qkv_kvlen_impl("dh_attn_decode_qkv_kvlen", false, d_qkv, d_q_weight, d_k_weight, d_cos, d_sin, d_cache_k,
                                    d_cache_v, d_O, H, Hkv, D, d_kv_len, max_kv_len, rotary_dim, interleaved, eps,
                                    weight_offset, use_norm, scale, softcap, sliding_window, kv_start, kv_layout, d_workspace);
}

int dh_attn_decode_qkv_kvlen_partials(const float* d_qkv, const float* d_q_weight, const float* d_k_weight,
                                      const float* d_cos, const float* d_sin, void* d_cache_k, void* d_cache_v, int H,
                                      int Hkv, int D, const uint32_t* d_kv_len, int max_kv_len, int rotary_dim,
                                      int interleaved, float eps, int weight_offset, int use_norm, float scale,
                                      float softcap, int sliding_window, int kv_start, int kv_layout, void* d_workspace) {
  return attn_decode_qkv_kvlen_impl("dh_attn_decode_qkv_kvlen_partials", true, d_qkv, d_q_weight, d_k_weight, d_cos, d_sin,
                                    d_cache_k, d_cache_v, nullptr, H, Hkv, D, d_kv_len, max_kv_len, rotary_dim, interleaved,
                                    eps, weight_offset, use_norm, scale, softcap, sliding_window, kv_start, kv_layout,
                                    d_workspace);
}

}  // extern "C"
