// Q4_K GEMV for a handful of activation rows (M = 3..8) in ONE pass over the weights, on the f16
// matrix cores of gfx950.
//
// y[m][n] = sum over super-blocks b of  d_b * sum_k (sc_s(k) q_k) x[m][k]  -  dmin_b * sum_s mn_s * (sum_{k in s} x[m][k])
//
// v_mfma_f32_16x16x32_f16 multiplies 16 weight rows x 32 weights (one sub-block) by 16 operand
// rows.  A weight enters as the exact integer sc * q <= 945 in the bits of an f16 subnormal (times
// 2^-24): two nibbles are isolated per 32-bit word and both are multiplied by the 6-bit scale with
// one 24-bit integer multiply.  An activation row enters as two operand rows, the f16 value of
// x * 2^(14-e) (e from the largest magnitude of the row inside the super-block column) and the f16
// value of what that leaves, so x keeps 22 bits; eight rows fill the sixteen operand rows.  The
// eight sub-blocks of a super-block chain into one accumulator.  The min term is a ninth, tiny
// product of the same shape: the eight sub-block sums of a row (high and low part again) against
// the eight 6-bit mins of a weight row.  d, dmin and the power of two come in once per super-block
// in f32.
//
// Work split: a workgroup of 16 waves owns 16-row tiles; a work unit is 16 weight rows x one
// super-block column (2304 bytes, fetched by the load unit straight into the wave's LDS ring).  The
// units of a workgroup, ordered column by column, are cut into 16 equal runs, one per wave, so a
// wave meets few columns and converts each of them itself, in registers: no wave ever waits for
// another one.  Every lane loads 4 consecutive activations per sub-block (the raw values of the next
// column are requested while the last unit of the current one is multiplied: the operand of a
// sub-block is spent after its product, and its registers take the load), and lane pairs swap
// halves so that the high-part row and the low-part row of an activation row each see all 8 values
// of their k-group.  Partial sums of a wave's units go to private LDS accumulators, one per (tile,
// matrix); after one barrier at the end the sixteen waves' accumulators are added in wave order
// (deterministic) and the outputs written.
#include <algorithm>
#include <type_traits>
#include <cstdlib>

#include "dh_common.h"
#include "q4k_device.h"

namespace {

using dh::kBlockBytes;
using dh::kQK;

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef uint32_t v2u __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

constexpr int kWaves = 16;
constexpr int kTileRows = 16;
constexpr int kStage = kTileRows * kBlockBytes;   // 2304 bytes per ring stage
constexpr int kUnitLoads = 3;                     // load instructions of a full unit: ceil(16 rows * 9 pieces / 64 lanes)
constexpr int kMaxDepth = 2;
constexpr int kAccBytes = 512;                    // one accumulator: 64 lanes x 2 floats
constexpr size_t kMaxLds = 160 * 1024;
constexpr size_t kLdsCap = kMaxLds;
constexpr int kSsqFloats = 16;                    // per wave: the sums of squares of the 8 activation rows (RMSNorm prologue), pad

#define DH_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
// s_waitcnt with only the vector-memory counter set (6 bits, split 4 + 2 in the encoding).
#define DH_WAIT_VM(k) __builtin_amdgcn_s_waitcnt(((k) & 0xF) | (((k) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

// Waits until at most n of this wave's vector-memory loads are outstanding (loads complete in
// issue order).  Counts without a case wait for everything, which is always safe.
__device__ __forceinline__ void wait_vm_at_most(int n) {
  switch (n) {
    case 1: DH_WAIT_VM(1); break;
    case 2: DH_WAIT_VM(2); break;
    case 3: DH_WAIT_VM(3); break;
    case 4: DH_WAIT_VM(4); break;
    case 5: DH_WAIT_VM(5); break;
    case 6: DH_WAIT_VM(6); break;
    default: DH_WAIT_VM(0); break;
  }
}

struct RowsArgs {
  const float* A;        // [M][K] f32, or f16 in the AF16 kernels
  const uint8_t* W;      // Q4_K rows
  const uint8_t* W2;     // second matrix (DUAL) or null
  void* C;               // [M][N] f32 or f16
  const float* residual; // [M][N] or null
  const float* norm_weight;   // RMSNorm prologue (null = off)
  int M, N, K, nb;
  int depth;             // ring stages per wave
  int rows;              // weight rows per tile (<= 16), chosen so that the tiles divide evenly among the workgroups
  int nlw;               // load instructions per unit: ceil(9 * rows / 64)
  int grid;              // workgroups launched
  int tiles_base, tiles_rem;   // tiles per workgroup: floor and remainder of tiles / grid
  int acc_max;           // accumulators per wave the LDS block was sized for: (tiles_base + 1 if tiles_rem) * matrices
  int c_f16, activation, norm_weight_offset;
  float alpha, clamp_max, norm_eps;
};

// value of lane ^ 1
__device__ __forceinline__ uint32_t swap_pair_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, 0xB1, 0xF, 0xF, false);   // quad_perm [1,0,3,2]
}
__device__ __forceinline__ float swap_pair_f32(float v) { return __uint_as_float(swap_pair_u32(__float_as_uint(v))); }

// Sum / largest over the eight lanes that share an activation row: lane ^ 1 and the four 16-lane rows.
__device__ __forceinline__ float row_lanes_sum(float v) {
  v += swap_pair_f32(v);
  const uint32_t u = __float_as_uint(v);
  auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const uint32_t w = __float_as_uint(v);
  auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}
__device__ __forceinline__ float row_lanes_max(float v) {
  v = fmaxf(v, swap_pair_f32(v));
  const uint32_t u = __float_as_uint(v);
  auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const uint32_t w = __float_as_uint(v);
  auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

__device__ __forceinline__ uint32_t mul24(uint32_t a, uint32_t b) { return (uint32_t)__umul24(a, b); }
__device__ __forceinline__ uint32_t pack_f16_rtz(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
}
__device__ __forceinline__ float f16_bits_lo(uint32_t v) { return (float)__builtin_bit_cast(_Float16, (unsigned short)(v & 0xffffu)); }
__device__ __forceinline__ float f16_bits_hi(uint32_t v) { return (float)__builtin_bit_cast(_Float16, (unsigned short)(v >> 16)); }

// One column's operands in the registers of a wave.  Lane (i = lane & 15, kg = lane >> 4) is operand
// row i = 2 r + part (activation row r, part 0 = high, 1 = low) and k-group kg.
struct ColOps {
  v4u xa[8];       // one operand per sub-block
  uint32_t xm;     // first word of the min term's operand (the other three are zero): slots 0, 1 of k-group kg
                   // = sums of sub-blocks 2 (kg & 1) + 4 (kg >> 1) and the next
  float xinv0, xinv1;   // 2^24 / scale of activation rows 2 kg, 2 kg + 1
};

// Dynamic LDS block, in this order:
//   ring  [16 waves][depth][2304]
//   wn    [16 waves][256] floats: RMSNorm weights of the column being converted (norm prologue only)
//   ssq   [16 waves][kSsqFloats]: the wave's sum of squares of activation row r at r
//   acc   [16 waves][acc_max][64 lanes][2]: lane (j, kg) keeps weight row j x activation rows 2 kg, 2 kg + 1
template <bool DUAL, bool VEC, bool AF16 = false>
__global__ __launch_bounds__(64 * kWaves, 1) void q4k_gemv_rows_kernel(const RowsArgs a) {
  constexpr int NMAT = DUAL ? 2 : 1;
  extern __shared__ __align__(16) unsigned char lds[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // the arguments the streaming loop uses are fetched in one batch (left alone the compiler fetches
  // some of them only where they are first used: a second, dependent trip to memory)
  asm volatile("" :: "s"(a.A), "s"(a.W), "s"(a.W2), "s"(a.norm_weight));
  asm volatile("" :: "s"(a.M), "s"(a.N), "s"(a.K), "s"(a.nb), "s"(a.depth), "s"(a.rows), "s"(a.nlw), "s"(a.grid),
               "s"(a.tiles_base), "s"(a.tiles_rem), "s"(a.acc_max));

  const int D = a.depth, nb = a.nb;
  const bool norm = a.norm_weight != nullptr;
  unsigned char* ring = lds;
  float* wn = reinterpret_cast<float*>(ring + (size_t)kWaves * D * kStage);
  float* ssq_lds = wn + (norm ? kWaves * kQK : 0);
  float* acc = ssq_lds + kWaves * kSsqFloats;

  const int64_t row_bytes = (int64_t)nb * kBlockBytes;
  const int ntl = a.tiles_base + ((int)blockIdx.x < a.tiles_rem ? 1 : 0);   // this workgroup's tiles: blockIdx.x + i * grid
  const int nacc = ntl * NMAT;
  const int total = nb * nacc;                 // units of the workgroup, ordered (column, tile, matrix)
  const int q0 = (wave * total) >> 4, q1 = ((wave + 1) * total) >> 4;
  const int nun = q1 - q0;                     // this wave's run
  unsigned char* my_ring = ring + (size_t)wave * D * kStage;
  float* my_acc = acc + (size_t)wave * a.acc_max * 128;
  const uint32_t acc_abs = (uint32_t)(uintptr_t)DH_LDS_PTR(my_acc);

  // nothing is in flight yet: plain stores
  for (int i = 0; i < nacc; i++) reinterpret_cast<float2*>(my_acc)[i * 64 + lane] = make_float2(0.f, 0.f);
  if (lane < kSsqFloats) ssq_lds[wave * kSsqFloats + lane] = 0.f;

  // piece p = t*64 + lane of a unit: row p/9, 16-byte piece p%9 of that row's super-block; kept as
  // row + 256 * (byte offset of the piece), all ones for lanes past the tile's rows
  uint32_t gpiece[kUnitLoads];
#pragma unroll
  for (int t = 0; t < kUnitLoads; t++) {
    const int p = t * 64 + lane, r = p / 9;
    gpiece[t] = p < 9 * a.rows ? (uint32_t)(r + 256 * 16 * (p - r * 9)) : 0xFFFFFFFFu;
  }
  const uint32_t row_bytes32 = (uint32_t)row_bytes;     // a tile spans at most 16 rows: offsets inside it fit 32 bits

  // Puts the loads of the unit (column col_, accumulator acc_ = tile ordinal * NMAT + matrix) in flight into ring
  // stage stage_.  Rows past the end of the matrix (last tile) read the last row again.
#define DH_ISSUE(col_, acc_, stage_)                                                              \
  do {                                                                                            \
    const int itl_ = DUAL ? (acc_) >> 1 : (acc_);                                                 \
    const int imat_ = DUAL ? (acc_) & 1 : 0;                                                      \
    const int tile_ = (int)blockIdx.x + itl_ * a.grid;                                            \
    const uint8_t* base_ = ((DUAL && imat_) ? a.W2 : a.W) + (int64_t)tile_ * a.rows * row_bytes + \
                           (int64_t)(col_) * kBlockBytes;                                         \
    unsigned char* st_ = my_ring + (stage_) * kStage;                                             \
    const uint32_t last_ = (uint32_t)(a.N - tile_ * a.rows - 1);                                  \
    _Pragma("unroll") for (int t = 0; t < kUnitLoads; t++) {                                      \
      if (gpiece[t] != 0xFFFFFFFFu) {                                                             \
        const uint32_t o_ = min(gpiece[t] & 0xFFu, last_) * row_bytes32 + (gpiece[t] >> 8);       \
        __builtin_amdgcn_global_load_lds(base_ + o_, DH_LDS_PTR(st_ + t * 1024), 16, 0, 0);       \
      }                                                                                           \
    }                                                                                             \
  } while (0)

  // ---- activation side.  For sub-block s the lane loads the 4 activations
  // 256 col + 32 s + 8 kg + 4 part .. + 3 of its row.  The loads are hand-written instructions (scalar
  // base + 32-bit lane offset), so the compiler believes them complete at once: the raw registers
  // are declared where they are loaded and only straight-line code lies between the load and the
  // wait, which leaves it no reason to move them earlier.  The s_nop in front of each load is not
  // padding: a vector-memory instruction must not read a scalar register within five wait states of a
  // vector instruction writing it (v_readlane restoring a spilled scalar, v_readfirstlane), the compiler
  // keeps that distance only for instructions it emits itself, and a build under scalar-register
  // pressure put such a restore of the activation pointer directly in front of one of these loads: the
  // load then went to a wild address.
  const int kg = lane >> 4, j = lane & 15;
  const int xrow = j >> 1, part = j & 1;
  const int xk = 8 * kg + 4 * part;             // offset of the lane's 4 activations inside a sub-block
  const bool row_ok = xrow < a.M;
  const float* xbase = a.A + (int64_t)min(xrow, a.M - 1) * a.K;
  // (f16 rows: two bytes per element, the lane's four elements are two registers, widened where they are converted)
  constexpr uint32_t XB = AF16 ? 2u : 4u;
  using XRaw = std::conditional_t<AF16, v2u, v4f>;
  const uint32_t xrow_off = XB * (uint32_t)(min(xrow, a.M - 1) * a.K);     // M K stays far below 2^30 (M <= 8)
  const uint32_t wn_lane = (uint32_t)(uintptr_t)DH_LDS_PTR(wn + wave * kQK) + 4 * xk;   // this lane's norm weights of sub-block 0
#define DH_LOAD_X_ONE(xr_, col_, s_)                                                              \
  do {                                                                                            \
    const int k_ = (col_) * kQK + 32 * (s_) + xk;                                                 \
    if constexpr (AF16) {                                                                         \
      const uint32_t o_ = xrow_off + XB * (uint32_t)min(k_, a.K - 4);                             \
      asm volatile("s_nop 4\n\tglobal_load_dwordx2 %0, %1, %2" : "=&v"((xr_)[s_]) : "v"(o_), "s"(a.A) : "memory"); \
    } else if constexpr (VEC) {                                                                   \
      const uint32_t o_ = xrow_off + XB * (uint32_t)min(k_, a.K - 4);                             \
      asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2" : "=&v"((xr_)[s_]) : "v"(o_), "s"(a.A) : "memory"); \
    } else {                                                                                      \
      _Pragma("unroll") for (int e = 0; e < 4; e++) (xr_)[s_][e] = xbase[min(k_ + e, a.K - 1)];   \
    }                                                                                             \
  } while (0)
  // the column's RMSNorm weights, 16 bytes per lane, straight into the wave's LDS area
#define DH_LOAD_NORM_WEIGHTS(col_)                                                                \
  do {                                                                                            \
    if (VEC && norm) {                                                                            \
      const int k_ = (col_) * kQK + 4 * lane;                                                     \
      __builtin_amdgcn_global_load_lds(a.norm_weight + min(k_, a.K - 4), DH_LDS_PTR(wn + wave * kQK), 16, 0, 0); \
    }                                                                                             \
  } while (0)

  float ssq = 0.f;                              // this lane's share of the sum of squares of row xrow
  // Turns the raw activations xr of column col into operands.  count: the column's squares go into
  // this wave's sum (the wave that holds the column's first unit counts them).
  auto convert = [&](XRaw (&xraw)[8], const int col, const bool count, ColOps& out) __attribute__((always_inline)) {
    v4f xwide[8];
    if constexpr (AF16) {
#pragma unroll
      for (int s = 0; s < 8; s++)
        xwide[s] = v4f{f16lo(xraw[s].x), f16hi(xraw[s].x), f16lo(xraw[s].y), f16hi(xraw[s].y)};
    }
    v4f (&xr)[8] = *[&]() {
      if constexpr (AF16) return &xwide; else return &xraw;
    }();
    const bool tail = col * kQK + kQK > a.K;          // the column reaches past K: those elements count as zero
    float mx = 0.f;
    if (norm) {
      v4f w[8];
      if constexpr (VEC) {
        asm volatile(
            "ds_read_b128 %0, %8\n\t"
            "ds_read_b128 %1, %8 offset:128\n\t"
            "ds_read_b128 %2, %8 offset:256\n\t"
            "ds_read_b128 %3, %8 offset:384\n\t"
            "ds_read_b128 %4, %8 offset:512\n\t"
            "ds_read_b128 %5, %8 offset:640\n\t"
            "ds_read_b128 %6, %8 offset:768\n\t"
            "ds_read_b128 %7, %8 offset:896\n\t"
            "s_waitcnt lgkmcnt(0)"
            : "=&v"(w[0]), "=&v"(w[1]), "=&v"(w[2]), "=&v"(w[3]), "=&v"(w[4]), "=&v"(w[5]), "=&v"(w[6]), "=&v"(w[7])
            : "v"(wn_lane)
            : "memory");
      } else {
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
          for (int e = 0; e < 4; e++) w[s][e] = a.norm_weight[min(col * kQK + 32 * s + xk + e, a.K - 1)];
      }
      const float one = a.norm_weight_offset ? 1.0f : 0.0f;
      float sq = 0.f;
#pragma unroll
      for (int s = 0; s < 8; s++) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
          float v = xr[s][e];
          if (tail && col * kQK + 32 * s + xk + e >= a.K) v = 0.f;
          sq = fmaf(v, v, sq);
          xr[s][e] = v * (one + w[s][e]);
        }
      }
      if (count) ssq += sq;
    } else if (tail) {
#pragma unroll
      for (int s = 0; s < 8; s++)
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (col * kQK + 32 * s + xk + e >= a.K) xr[s][e] = 0.f;
    }
    // (one instruction per two elements; written through fmaxf/fabsf the compiler spends four)
#pragma unroll
    for (int s = 0; s < 8; s++) {
      asm("v_max3_f32 %0, %0, |%1|, |%2|" : "+v"(mx) : "v"(xr[s][0]), "v"(xr[s][1]));
      asm("v_max3_f32 %0, %0, |%1|, |%2|" : "+v"(mx) : "v"(xr[s][2]), "v"(xr[s][3]));
    }
    mx = row_lanes_max(mx);
    int ex = (int)((__float_as_uint(mx) >> 23) & 0xFF) - 127;      // mx < 2^(ex+1)
    // The factors 2^(14 - ex) and 2^(10 + ex) must both be normal numbers.  Rows whose largest magnitude
    // is 2^118 or more (or infinite) overflow the f16 operands and come out non-finite; a NaN
    // activation is no maximum (v_max3 skips it) and travels through the matrix core as NaN.
    ex = max(-112, min(117, ex));
    if (mx == 0.f) ex = 0;
    // |x| sf < 2^15; rows past M become zero operands
    const float sf = row_ok ? __uint_as_float((uint32_t)(127 + 14 - ex) << 23) : 0.f;
    float p[8];
#pragma unroll
    for (int s = 0; s < 8; s++) {
      const float t0 = xr[s][0] * sf, t1 = xr[s][1] * sf, t2 = xr[s][2] * sf, t3 = xr[s][3] * sf;
      // operand slots follow the masked weight words: (byte 0, byte 2), (byte 1, byte 3)
      const uint32_t h02 = pack_f16_rtz(t0, t2), h13 = pack_f16_rtz(t1, t3);
      const uint32_t l02 = pack_f16_rtz(t0 - f16_bits_lo(h02), t2 - f16_bits_hi(h02));
      const uint32_t l13 = pack_f16_rtz(t1 - f16_bits_lo(h13), t3 - f16_bits_hi(h13));
      // the high-part lane holds elements 0..3 and wants the partner's high parts of 4..7; the
      // low-part lane holds 4..7 and wants the partner's low parts of 0..3
      const uint32_t r0 = swap_pair_u32(part ? h02 : l02), r1 = swap_pair_u32(part ? h13 : l13);
      out.xa[s] = part ? v4u{r0, r1, l02, l13} : v4u{h02, h13, r0, r1};
      p[s] = (xr[s][0] + xr[s][1]) + (xr[s][2] + xr[s][3]);
    }
    // Sub-block sums over the row's eight lanes, halving the values at every step: afterwards lane
    // (part, kg) holds the sum of sub-block part + 2 (kg & 1) + 4 (kg >> 1).
    float r4[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const float keep = part ? p[2 * i + 1] : p[2 * i], send = part ? p[2 * i] : p[2 * i + 1];
      r4[i] = keep + swap_pair_f32(send);
    }
    float t2[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
      // after the swap: even 16-lane rows hold (own first, partner's first), odd rows (partner's second, own second)
      auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(r4[2 * i]), __float_as_uint(r4[2 * i + 1]), false, false);
      t2[i] = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
    }
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(t2[0]), __float_as_uint(t2[1]), false, false);
    const float sum = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
    {
      // min-term operand: high and low part of the sum (a sum stays below 32 x the largest element);
      // the row's high-part lane takes both high parts (its own sub-block in slot 0, the partner's in
      // slot 1), the low-part lane both low parts
      const float t = sum * (sf * 0.03125f);
      const uint32_t hq = pack_f16_rtz(t, 0.f);
      const uint32_t lq = pack_f16_rtz(t - f16_bits_lo(hq), 0.f);
      const uint32_t got = swap_pair_u32(part ? hq : lq);
      out.xm = part ? ((got & 0xffffu) | (lq << 16)) : ((hq & 0xffffu) | (got << 16));
    }
    // 2^24 / sf of every row (lane 2 r holds row r's), then this lane's two
    const int xi = (127 + 10 + ex) << 23;
    const float e0 = __int_as_float(__builtin_amdgcn_readlane(xi, 0)), e1 = __int_as_float(__builtin_amdgcn_readlane(xi, 2));
    const float e2 = __int_as_float(__builtin_amdgcn_readlane(xi, 4)), e3 = __int_as_float(__builtin_amdgcn_readlane(xi, 6));
    const float e4 = __int_as_float(__builtin_amdgcn_readlane(xi, 8)), e5 = __int_as_float(__builtin_amdgcn_readlane(xi, 10));
    const float e6 = __int_as_float(__builtin_amdgcn_readlane(xi, 12)), e7 = __int_as_float(__builtin_amdgcn_readlane(xi, 14));
    out.xinv0 = kg == 0 ? e0 : kg == 1 ? e2 : kg == 2 ? e4 : e6;
    out.xinv1 = kg == 0 ? e1 : kg == 1 ? e3 : kg == 2 ? e5 : e7;
  };

  // ---- cursors: (column, accumulator) of the unit consumed next / issued next
  int colc = 0, accc = 0;
  if (nun > 0) {
    colc = q0 / nacc;
    accc = q0 - colc * nacc;
  }
  int coli = colc, acci = accc;
  int issued = 0, consumed = 0;
  ColOps cur;
#pragma unroll
  for (int s = 0; s < 8; s++) cur.xa[s] = v4u{0u, 0u, 0u, 0u};
  cur.xm = 0u;
  cur.xinv0 = cur.xinv1 = 0.f;
  if (nun > 0) {
    XRaw xr[8];
#pragma unroll
    for (int s = 0; s < 8; s++) DH_LOAD_X_ONE(xr, colc, s);
    DH_LOAD_NORM_WEIGHTS(colc);
    for (int d = 0; d < D; d++) {
      if (issued < nun) {
        DH_ISSUE(coli, acci, d);
        issued++;
        if (++acci == nacc) { acci = 0; coli++; }
      }
    }
    // only the activations are waited for (the units were requested behind them)
    if constexpr (VEC) wait_vm_at_most(issued * a.nlw); else DH_WAIT_VM(0);
#pragma unroll
    for (int s = 0; s < 8; s++) asm volatile("" : "+v"(xr[s]));
    convert(xr, colc, accc == 0, cur);
  }

  const uint32_t lane_hdr = (uint32_t)(uintptr_t)DH_LDS_PTR(my_ring) + (uint32_t)j * kBlockBytes;
  const uint32_t lane_q = lane_hdr + 16 + 8 * kg;
  // the min term's weight-side operand takes the mins of sub-blocks 2 (kg & 1) + 4 (kg >> 1) and the next
  const uint32_t mn_shift = 16u * (uint32_t)(kg & 1);

  int cstage = 0;
  // One unit; SW: the next unit starts column coln, whose activations are requested while this unit is
  // multiplied and converted at the end.
  auto unit = [&](auto sw_tag, const int coln) __attribute__((always_inline)) {
    constexpr bool SW = decltype(sw_tag)::value;
    XRaw xr[8];
    wait_vm_at_most((issued - consumed - 1) * a.nlw);
    const uint32_t hp = lane_hdr + cstage * kStage, qp = lane_q + cstage * kStage;
    v4u h;
    v2u q[4];
    v2f run;                                 // the accumulator this unit adds to (private to the wave)
    const uint32_t accp = acc_abs + (uint32_t)accc * kAccBytes + 8 * lane;
    // (all LDS reads while weights are in flight are hand-written: the compiler would put a wait for
    // every load in flight in front of its own, because those loads write LDS too)
    asm volatile(
        "ds_read_b128 %0, %6\n\t"
        "ds_read_b64 %1, %7\n\t"
        "ds_read_b64 %2, %7 offset:32\n\t"
        "ds_read_b64 %3, %7 offset:64\n\t"
        "ds_read_b64 %4, %7 offset:96\n\t"
        "ds_read_b64 %5, %8\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(h), "=&v"(q[0]), "=&v"(q[1]), "=&v"(q[2]), "=&v"(q[3]), "=&v"(run)
        : "v"(hp), "v"(qp), "v"(accp)
        : "memory");
    // the stage is free again: the unit `depth` ahead goes into it.  Before a new column that waits
    // until the column's activations have been requested: loads complete in issue order, and the
    // activations must not queue behind a unit.
    const bool issued_now = issued < nun;
    if (!SW && issued_now) {
      DH_ISSUE(coli, acci, cstage);
      issued++;
      if (++acci == nacc) { acci = 0; coli++; }
    }

    // all eight 6-bit scales / mins of this lane's weight row, one byte each
    const uint32_t sc_lo4 = h.y & 0x3F3F3F3Fu;
    const uint32_t mn_lo4 = h.z & 0x3F3F3F3Fu;
    const uint32_t sc_hi4 = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
    const uint32_t mn_hi4 = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
    v4f dd = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 4; c++) {
#pragma unroll
      for (int p = 0; p < 2; p++) {
        const int s = 2 * c + p;
        const uint32_t w0 = p ? q[c].x >> 4 : q[c].x, w1 = p ? q[c].y >> 4 : q[c].y;
        const uint32_t sc = ((s < 4 ? sc_lo4 : sc_hi4) >> (8 * (s & 3))) & 0xFFu;
        // two weights per word, each times the scale: products stay below 2^10, inside their 16-bit fields
        const v4u b = {mul24(w0 & 0x000F000Fu, sc), mul24((w0 >> 8) & 0x000F000Fu, sc),
                       mul24(w1 & 0x000F000Fu, sc), mul24((w1 >> 8) & 0x000F000Fu, sc)};
        dd = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, cur.xa[s]), __builtin_bit_cast(half8_t, b),
                                                    dd, 0, 0, 0);
        if constexpr (SW) {
          // the operand of this sub-block is spent: its registers can take the next column's raw values
          DH_LOAD_X_ONE(xr, coln, s);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    if constexpr (SW) DH_LOAD_NORM_WEIGHTS(coln);
    // the min term: the two mins that belong to this lane's k-group, in the same subnormal integer form
    v4f dm;
    {
      const uint32_t two = (kg >> 1 ? mn_hi4 : mn_lo4) >> mn_shift;
      const v4u b = {__builtin_amdgcn_perm(0u, two, 0x0c010c00u), 0u, 0u, 0u};
      const v4u xm4 = {cur.xm, 0u, 0u, 0u};
      dm = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, xm4), __builtin_bit_cast(half8_t, b),
                                                  v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
    }
    // lane (j, kg): dd[0..3] = operand rows 4 kg .. 4 kg + 3 = activation rows 2 kg, 2 kg + 1, high and low parts
    const float d = f16lo(h.x), dmin32 = 32.0f * f16hi(h.x);
    // (a read, an add and a write: LDS float atomics are far slower)
    run[0] += cur.xinv0 * fmaf(d, dd[0] + dd[1], -dmin32 * (dm[0] + dm[1]));
    run[1] += cur.xinv1 * fmaf(d, dd[2] + dd[3], -dmin32 * (dm[2] + dm[3]));
    asm volatile("ds_write_b64 %0, %1" :: "v"(accp), "v"(run) : "memory");
    if (SW && issued_now) {
      DH_ISSUE(coli, acci, cstage);
      issued++;
      if (++acci == nacc) { acci = 0; coli++; }
    }
    cstage = cstage + 1 == D ? 0 : cstage + 1;
    consumed++;
    if constexpr (SW) {
      // the activations were requested after every older unit and before the one just issued
      if constexpr (VEC) wait_vm_at_most(issued_now ? a.nlw : 0); else DH_WAIT_VM(0);
#pragma unroll
      for (int s = 0; s < 8; s++) asm volatile("" : "+v"(xr[s]));
      convert(xr, coln, true, cur);
    }
  };
#pragma unroll 1
  while (consumed < nun) {
    int coln = colc, accn = accc + 1;
    if (accn == nacc) { accn = 0; coln++; }
    if (consumed + 1 < nun && coln != colc)
      unit(std::true_type{}, coln);
    else
      unit(std::false_type{}, coln);
    colc = coln;
    accc = accn;
  }
#undef DH_ISSUE
#undef DH_LOAD_X_ONE
#undef DH_LOAD_NORM_WEIGHTS

  // ---- the wave's sums of squares (RMSNorm prologue), then everybody meets
  if (norm) {
    const float t = row_lanes_sum(ssq);
    if (part == 0 && kg == 0)
      asm volatile("ds_write_b32 %0, %1" :: "v"((uint32_t)(uintptr_t)DH_LDS_PTR(ssq_lds + wave * kSsqFloats) + 4 * xrow), "v"(t) : "memory");
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");

  // ---- outputs: element e of an accumulator = lane (j, kg) x row 2 kg + (e & 1); the sixteen waves' values in wave order
  for (int idx = tid; idx < ntl * 128; idx += 64 * kWaves) {
    const int tl = idx >> 7, e = idx & 127;
    const int ol = e >> 1, oj = ol & 15, m = 2 * (ol >> 4) + (e & 1);
    float sg = 0.f, su = 0.f;
#pragma unroll 4
    for (int w = 0; w < kWaves; w++) {
      const float* p = acc + ((size_t)w * a.acc_max + tl * NMAT) * 128 + e;
      sg += p[0];
      if (DUAL) su += p[128];
    }
    if (norm) {
      float tot = 0.f;
      for (int w = 0; w < kWaves; w++) tot += ssq_lds[w * kSsqFloats + m];
      const float inv = 1.0f / sqrtf(tot / (float)a.K + a.norm_eps);
      sg *= inv;
      su *= inv;
    }
    const int tile = (int)blockIdx.x + tl * a.grid;
    const int64_t row = (int64_t)tile * a.rows + oj;
    if (oj < a.rows && m < a.M && row < a.N) {
      float v;
      if (DUAL) {
        const float act = a.activation == DH_ACT_SILU ? act_silu(sg) : act_gelu(sg);
        v = act * su * a.alpha;
        if (a.activation == DH_ACT_SILU && a.clamp_max > 0.f) v = fminf(fmaxf(v, -a.clamp_max), a.clamp_max);
      } else {
        v = sg * a.alpha;
        if (a.residual) v += a.residual[(int64_t)m * a.N + row];
      }
      if (a.c_f16)
        reinterpret_cast<__half*>(a.C)[(int64_t)m * a.N + row] = __float2half(v);
      else
        reinterpret_cast<float*>(a.C)[(int64_t)m * a.N + row] = v;
    }
  }
}

int env_int(const char* name, int dflt) { return dh::tuning_int(name, dflt); }

template <bool DUAL, bool VEC, bool AF16 = false>
int launch_rows(RowsArgs a, const char* op) {
  constexpr int NMAT = DUAL ? 2 : 1;
  auto kern = q4k_gemv_rows_kernel<DUAL, VEC, AF16>;
  const int ncu = dh::num_cus();
  // rows per tile: the largest count <= 16 that gives every workgroup the same number of tiles
  const int per_cu = (int)dh::ceil_div(a.N, (int64_t)ncu * kTileRows);
  a.rows = std::max(1, std::min(kTileRows, (int)dh::ceil_div(a.N, (int64_t)ncu * per_cu)));
  a.nlw = (9 * a.rows + 63) / 64;
  const int64_t ntiles = dh::ceil_div(a.N, a.rows);
  const int grid = (int)std::min<int64_t>(ntiles, ncu);
  a.grid = grid;
  a.tiles_base = (int)(ntiles / grid);
  a.tiles_rem = (int)(ntiles % grid);
  a.acc_max = (a.tiles_base + (a.tiles_rem ? 1 : 0)) * NMAT;
  // about a run per wave: with far fewer units than waves most of the workgroup idles, and the
  // kernel that spreads a tile's columns over the waves is faster (measured on 1024 x 3072 and smaller)
  static const int env_min_units = env_int("DH_GEMV_ROWS_MIN_UNITS", 12);
  if ((int64_t)a.nb * a.tiles_base * NMAT < env_min_units) return -1;
  auto lds_for = [&](int dep) {
    return (size_t)kWaves * dep * kStage + (a.norm_weight ? sizeof(float) * kWaves * kQK : 0) +
           sizeof(float) * kWaves * kSsqFloats + (size_t)kWaves * a.acc_max * kAccBytes;
  };
  static const int env_depth = env_int("DH_GEMV_ROWS_DEPTH", 0);
  int depth = env_depth > 0 ? std::min(kMaxDepth, env_depth) : kMaxDepth;
  while (depth > 1 && lds_for(depth) > kLdsCap) depth--;
  if (lds_for(depth) > kLdsCap) return -1;
  a.depth = depth;
  {
    const int64_t rec[12] = {a.rows, a.nlw, grid, a.tiles_base, a.tiles_rem, depth, (int64_t)lds_for(depth), 0, 0, 0, a.acc_max,
                             a.M};
    for (int i = 0; i < 12; i++) dh::plan_layout(i, rec[i]);
  }
  if (dh::plan_note(DH_PLAN_GEMV_ROWS)) return 0;
  static bool attr_set = false;   // once per instantiation: the call costs microseconds
  if (!attr_set) {
    DH_CHECK_HIP(op, hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsCap));
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * kWaves), lds_for(depth), dh::stream(), a);
  DH_CHECK_LAUNCH(op);
  return 0;
}

}  // namespace

namespace dh {

int q4k_gemv_rows(const char* op, const float* A, const uint8_t* W, const uint8_t* W2, void* C, int c_f16,
                  const float* residual, int M, int N, int K, float alpha, int activation, float clamp_max,
                  const float* norm_weight, float norm_eps, int norm_weight_offset, int a_f16) {
  static const int off = env_int("DH_GEMV_ROWS_OFF", 0);
  if (off || M < 1 || M > 8) return -1;
  RowsArgs a{};
  a.A = A; a.W = W; a.W2 = W2; a.C = C; a.residual = residual;
  a.M = M; a.N = N; a.K = K; a.nb = (K + kQK - 1) / kQK;
  a.alpha = alpha; a.c_f16 = c_f16; a.activation = activation; a.clamp_max = clamp_max;
  a.norm_weight = norm_weight; a.norm_eps = norm_eps; a.norm_weight_offset = norm_weight_offset;
  const bool vec = (K & 3) == 0 && (reinterpret_cast<uintptr_t>(A) & 15) == 0 &&
                   (!norm_weight || (reinterpret_cast<uintptr_t>(norm_weight) & 15) == 0);
  if (a_f16) {
    // f16 rows: the single-matrix product without a norm prologue, K a multiple of 4, 8-byte aligned rows
    if (W2 || norm_weight || (K & 3) != 0 || (reinterpret_cast<uintptr_t>(A) & 7) != 0) return -1;
    return launch_rows<false, true, true>(a, op);
  }
  if (W2) return vec ? launch_rows<true, true>(a, op) : launch_rows<true, false>(a, op);
  return vec ? launch_rows<false, true>(a, op) : launch_rows<false, false>(a, op);
}

}  // namespace dh
