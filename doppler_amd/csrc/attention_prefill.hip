// Prefill attention (T query tokens at once) over an f16 KV cache with grouped-query heads, on the
// matrix cores: the flash-attention recurrence with v_mfma_f32_16x16x32_f16.
//
// Grid = (query tiles of 64 QT tokens, query heads); a workgroup is 4 waves, wave w owns QT
// groups of 16 consecutive query rows of the tile.  Keys advance 64 at a time; the K and V tiles
// of the head's kv head are staged in LDS once per workgroup and shared by the four waves, and
// every fragment a wave reads from there feeds QT matrix-core instructions (QT = 2 for prompts
// long enough to fill the compute units with 128-query tiles: the kernel is bound by
// instruction issue and LDS round trips per product, not by the matrix cores or by LDS
// bandwidth; 118 -> 102 us at T = 2048, 32 heads).
//
// Everything is computed transposed, so that the softmax statistics of a query live in the lanes
// that also hold its output column and nothing has to be shuffled between the two products:
//   S^T = K . Q^T   A = K rows from LDS (16 bytes of a key row per lane), B = Q^T from registers
//                   (scale folded in, rounded to f16).  D[key][q]: lane (q = l & 15, g = l >> 4)
//                   gets keys 16j + 4g + i (i < 4) of key subtile j.
//   softmax         per query = per lane column: maxima and sums over a lane's 16 values, the
//                   maxima then across the four lanes l, l+16, l+32, l+48 (lane-swap
//                   instructions), the sums only once after the last tile; fp32, online rescale.
//   O^T = V^T . P^T B = P^T is exactly the lane's own probabilities (k-slot (g, i') stands for
//                   key 16 (2 kb + i'/4) + 4g + i'%4 of 32-key block kb: a contraction index may be
//                   renumbered as long as both operands agree), A = V^T read from LDS, where the
//                   V tile was stored transposed with its keys in that same slot order.
// Causal tiles beyond the tile's last query are never visited.
// (Measured without effect at T = 2048..4096: a second LDS buffer per tile with one barrier per
// tile instead of two, and dispatching the long late-query tiles first.)
#include <algorithm>
#include <cfloat>
#include <cstdlib>

#include "dh_common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) _Float16 half8_t;
typedef __attribute__((ext_vector_type(4))) float float4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;   // plain vector type: arrays of it stay in registers

constexpr int BKEYS = 64;

// The four lanes l, l ^ 16, l ^ 32, l ^ 48 hold one query's scores.  v_permlane32_swap and
// v_permlane16_swap (gfx950) hand a lane its partner's value through the vector ALU: with both
// operands the same register, one result holds the lane's own half (row) pair and the other the
// partner's.  No LDS round trip, and no wait that would also stall on outstanding fragment reads.
__device__ __forceinline__ float quad_rows_max(float v) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float quad_rows_sum(float v) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

struct PrefillArgs {
  const float* Q;       // [T][H][D]
  const __half* K;      // [rows][Hkv][D]
  const __half* V;
  float* O;             // [T][H][D]
  int T, H, Hkv, G, kv_len, start_pos, causal, window;
  float scale, softcap;
};

// QT = 16-query groups per wave: every K and V fragment read from LDS feeds QT matrix-core
// instructions, and a workgroup tile (64 QT queries) stages each key tile once.
template <int D, int QT>
__global__ __launch_bounds__(256) void attn_prefill_kernel(const PrefillArgs a) {
  constexpr int BQ = 64 * QT;
  constexpr int STEPS = D / 32;            // MFMAs per 16 x 16 score tile
  constexpr int DT = D / 16;               // output row tiles (of O^T)
  constexpr int KROW = D + 8;              // halves per K row in LDS (16-byte pad)
  constexpr int VROW = BKEYS + 8;          // halves per V^T row in LDS
  constexpr int PIECES = BKEYS * D / 8 / 256;   // 16-byte pieces of a tile per thread
  __shared__ __align__(16) _Float16 k_lds[BKEYS * KROW];
  __shared__ __align__(16) _Float16 v_lds[D * VROW];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int q = lane & 15, g = lane >> 4;
  const int h = blockIdx.y, kvh = h / a.G;
  const int q0 = blockIdx.x * BQ;
  const int64_t kv_stride = (int64_t)a.Hkv * D;
  int my_q[QT], my_pos[QT];                                   // query token of this lane's column, its absolute position
#pragma unroll
  for (int u = 0; u < QT; u++) {
    my_q[u] = q0 + 16 * (QT * wave + u) + q;
    my_pos[u] = a.start_pos + my_q[u];
  }

  // ---- Q^T fragments (B operand): b[i] = scale * Q[my_q][32 s + 8 g + i].  Scores are kept in
  // units of log2(e), so that the softmax needs v_exp_f32 alone (with a soft cap the factor is
  // applied after the cap instead).
  constexpr float kLog2e = 1.4426950408889634f;
  const float qscale = a.softcap > 0.f ? a.scale : a.scale * kLog2e;
  half8_t qb[QT][STEPS];
#pragma unroll
  for (int u = 0; u < QT; u++)
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
      const float* qp = a.Q + ((int64_t)min(my_q[u], a.T - 1) * a.H + h) * D + 32 * s + 8 * g;
      const float4 v0 = reinterpret_cast<const float4*>(qp)[0], v1 = reinterpret_cast<const float4*>(qp)[1];
      const float qv[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
      for (int i = 0; i < 8; i++) qb[u][s][i] = (_Float16)(qv[i] * qscale);
    }

  // ---- key range of this query tile
  const int last_q = min(q0 + BQ, a.T) - 1;
  int kend = a.kv_len;
  if (a.causal) kend = min(kend, a.start_pos + last_q + 1);
  int kbeg = 0;
  if (a.window > 0) kbeg = max(0, a.start_pos + q0 - a.window + 1);
  kbeg = kbeg / BKEYS * BKEYS;
  const int ntiles = (kend - kbeg + BKEYS - 1) / BKEYS;

  float4_t acc[QT][DT];
  float m_run[QT], l_run[QT];
#pragma unroll
  for (int u = 0; u < QT; u++) {
#pragma unroll
    for (int t = 0; t < DT; t++) acc[u][t] = {0.f, 0.f, 0.f, 0.f};
    m_run[u] = -FLT_MAX;
    l_run[u] = 0.f;
  }

  u32x4_t kreg[PIECES], vreg[PIECES];
  // K piece p = tid + 256 r of a tile: key p / (D/8), 8 consecutive dims starting at 8 (p % (D/8)).
  // V is fetched by key PAIRS, so that the transposed tile can be written in 32-bit words: item j
  // of a thread is keys 2 (tid % 32), 2 (tid % 32) + 1 and dims 8 c .. 8 c + 7, c = tid / 32 + 8 j
  // (vreg[2 j + s] holds key s of the pair).  The 32 pairs of a half wave land in 32 different
  // LDS banks.
  const int vpair = tid & 31, vcol = tid >> 5;
#define DH_PF_LOAD(tile_)                                                                        \
  _Pragma("unroll") for (int r = 0; r < PIECES; r++) {                                           \
    const int p_ = tid + 256 * r, key_ = p_ / (D / 8), c_ = p_ % (D / 8);                        \
    const int row_ = min(kbeg + (tile_) * BKEYS + key_, a.kv_len - 1);                           \
    kreg[r] = *reinterpret_cast<const u32x4_t*>(a.K + (int64_t)row_ * kv_stride + (int64_t)kvh * D + 8 * c_); \
    const int vrow_ = min(kbeg + (tile_) * BKEYS + 2 * vpair + (r & 1), a.kv_len - 1);           \
    vreg[r] = *reinterpret_cast<const u32x4_t*>(a.V + (int64_t)vrow_ * kv_stride + (int64_t)kvh * D + \
                                              8 * (vcol + 8 * (r >> 1)));                        \
  }
  if (ntiles > 0) { DH_PF_LOAD(0); }

  for (int kt = 0; kt < ntiles; kt++) {
    __syncthreads();                                   // the previous tile has been consumed
#pragma unroll
    for (int r = 0; r < PIECES; r++) {
      const int p = tid + 256 * r, key = p / (D / 8), c = p % (D / 8);
      *reinterpret_cast<u32x4_t*>(&k_lds[key * KROW + 8 * c]) = kreg[r];
    }
    // V^T with the keys in k-slot order: key = 32 kb + 16 jj + 4 gg + ii -> slot 32 kb + 8 gg + 4 jj + ii;
    // the two keys of a pair are neighbours there, one 32-bit word per dim
    {
      const int key0 = 2 * vpair;
      const int slot = 32 * (key0 >> 5) + 8 * ((key0 >> 2) & 3) + 4 * ((key0 >> 4) & 1) + (key0 & 3);
#pragma unroll
      for (int j = 0; j < PIECES / 2; j++) {
        const int c = vcol + 8 * j;
        const u32x4_t aw = vreg[2 * j];
        const u32x4_t bw = vreg[2 * j + 1];
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const uint32_t word = __builtin_amdgcn_perm(bw[e >> 1], aw[e >> 1], (e & 1) ? 0x07060302u : 0x05040100u);
          reinterpret_cast<uint32_t*>(v_lds)[((8 * c + e) * VROW + slot) >> 1] = word;
        }
      }
    }
    __syncthreads();
    if (kt + 1 < ntiles) { DH_PF_LOAD(kt + 1); }

    // ---- S^T for this wave's 16 QT queries against the 64 keys
    const int kbase = kbeg + kt * BKEYS;
    float4_t st[QT][4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
#pragma unroll
      for (int u = 0; u < QT; u++) st[u][j] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < STEPS; s++) {
        const half8_t ka = *reinterpret_cast<const half8_t*>(&k_lds[(16 * j + q) * KROW + 32 * s + 8 * g]);
#pragma unroll
        for (int u = 0; u < QT; u++) st[u][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qb[u][s], st[u][j], 0, 0, 0);
      }
    }
    // ---- mask, soft cap, online softmax (this lane: query my_q, keys kbase + 16 j + 4 g + i).
    // A tile that every query of a 16-query group sees completely needs no per-element masks.
    half8_t pb[QT][2];
    float alpha[QT];
    bool rescale = false;
#pragma unroll
    for (int u = 0; u < QT; u++) {
      const int grp_lo = a.start_pos + q0 + 16 * (QT * wave + u), grp_hi = grp_lo + 15;
      const bool full = kbase + BKEYS <= a.kv_len && (!a.causal || kbase + BKEYS - 1 <= grp_lo) &&
                        (a.window <= 0 || kbase > grp_hi - a.window);
      float mx = -FLT_MAX;
      if (full && !(a.softcap > 0.f)) {
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
          for (int i = 0; i < 4; i++) mx = fmaxf(mx, st[u][j][i]);
      } else {
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const int key = kbase + 16 * j + 4 * g + i;
            float s = st[u][j][i];
            if (a.softcap > 0.f) s = tanhf(s / a.softcap) * (a.softcap * kLog2e);
            bool ok = key < a.kv_len;
            if (a.causal) ok = ok && key <= my_pos[u];
            if (a.window > 0) ok = ok && key > my_pos[u] - a.window;
            s = ok ? s : -INFINITY;
            st[u][j][i] = s;
            mx = fmaxf(mx, s);
          }
      }
      mx = quad_rows_max(mx);
      const float m_new = fmaxf(m_run[u], mx);              // finite: m_run starts at -FLT_MAX
      alpha[u] = __builtin_amdgcn_exp2f(m_run[u] - m_new);
      float ps = 0.f;
#pragma unroll
      for (int j = 0; j < 4; j++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const float p = __builtin_amdgcn_exp2f(st[u][j][i] - m_new);   // 2^-inf = 0 for masked keys
          ps += p;
          pb[u][j >> 1][4 * (j & 1) + i] = (_Float16)p;
        }
      l_run[u] = l_run[u] * alpha[u] + ps;               // this lane's share: alpha is the query's, the sum is taken once at the end
      m_run[u] = m_new;
      rescale = rescale || __builtin_amdgcn_ballot_w64(alpha[u] != 1.0f) != 0;   // no new maximum: nothing to scale
    }
    // ---- O^T = alpha O^T + V^T P^T
#pragma unroll
    for (int t = 0; t < DT; t++) {
      if (rescale) {
#pragma unroll
        for (int u = 0; u < QT; u++) acc[u][t] *= alpha[u];
      }
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
        const half8_t va = *reinterpret_cast<const half8_t*>(&v_lds[(16 * t + q) * VROW + 32 * kb + 8 * g]);
#pragma unroll
        for (int u = 0; u < QT; u++) acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, pb[u][kb], acc[u][t], 0, 0, 0);
      }
    }
  }
#undef DH_PF_LOAD

  // ---- lane (q, g) holds O[my_q][16 t + 4 g + i]
#pragma unroll
  for (int u = 0; u < QT; u++) {
    const float l = quad_rows_sum(l_run[u]);
    if (my_q[u] < a.T) {
      const float inv = l > 0.f ? 1.0f / l : 0.f;
      float* op = a.O + ((int64_t)my_q[u] * a.H + h) * D + 4 * g;
#pragma unroll
      for (int t = 0; t < DT; t++)
        *reinterpret_cast<float4*>(op + 16 * t) =
            make_float4(acc[u][t][0] * inv, acc[u][t][1] * inv, acc[u][t][2] * inv, acc[u][t][3] * inv);
    }
  }
}

}  // namespace

extern "C" int dh_attn_prefill(const float* d_Q, const void* d_K, const void* d_V, float* d_O, int T, int H,
                               int Hkv, int D, int kv_len, float scale, int causal, int start_pos,
                               float softcap, int sliding_window) {
  const char* op = "dh_attn_prefill";
  DH_REQUIRE_INIT(op);
  if (T <= 0 || H <= 0 || Hkv <= 0 || D <= 0)
    return dh::fail(1, "[%s] seqLen/numHeads/numKVHeads/headDim must be positive", op);
  if (H % Hkv) return dh::fail(1, "[%s] numHeads=%d must be a multiple of numKVHeads=%d", op, H, Hkv);
  if (D != 64 && D != 128) return dh::fail(1, "[%s] headDim %d not supported (64, 128)", op, D);
  if (kv_len <= 0 || start_pos < 0 || sliding_window < 0)
    return dh::fail(1, "[%s] kvLen must be positive, startPos and slidingWindow non-negative", op);
  if (causal && start_pos + T > kv_len)
    return dh::fail(1, "[%s] startPos=%d + seqLen=%d exceeds kvLen=%d", op, start_pos, T, kv_len);
  if (!d_Q || !d_K || !d_V || !d_O) return dh::fail(1, "[%s] null pointer", op);
  if ((reinterpret_cast<uintptr_t>(d_K) | reinterpret_cast<uintptr_t>(d_V) | reinterpret_cast<uintptr_t>(d_Q) |
       reinterpret_cast<uintptr_t>(d_O)) & 15)
    return dh::fail(1, "[%s] Q/K/V/O pointers must be 16-byte aligned", op);
  PrefillArgs a{};
  a.Q = d_Q; a.K = static_cast<const __half*>(d_K); a.V = static_cast<const __half*>(d_V); a.O = d_O;
  a.T = T; a.H = H; a.Hkv = Hkv; a.G = H / Hkv; a.kv_len = kv_len; a.start_pos = start_pos;
  a.causal = causal ? 1 : 0; a.window = sliding_window; a.scale = scale; a.softcap = softcap;
  // Two 16-query groups per wave (128 queries per workgroup) halve the LDS traffic per product;
  // short prompts keep 64-query tiles so that the grid still covers the compute units.
  static const int env_qt = dh::tuning_int("DH_ATTN_PREFILL_QT", 0);
  const int qt = env_qt ? env_qt : ((int64_t)dh::ceil_div(T, 128) * H >= 2 * dh::num_cus() ? 2 : 1);
  const dim3 grid((unsigned)dh::ceil_div(T, 64 * qt), (unsigned)H);
  if (D == 64) {
    if (qt == 2) hipLaunchKernelGGL((attn_prefill_kernel<64, 2>), grid, dim3(256), 0, dh::stream(), a);
    else hipLaunchKernelGGL((attn_prefill_kernel<64, 1>), grid, dim3(256), 0, dh::stream(), a);
  } else {
    if (qt == 2) hipLaunchKernelGGL((attn_prefill_kernel<128, 2>), grid, dim3(256), 0, dh::stream(), a);
    else hipLaunchKernelGGL((attn_prefill_kernel<128, 1>), grid, dim3(256), 0, dh::stream(), a);
  }
  DH_CHECK_LAUNCH(op);
  return 0;
}
