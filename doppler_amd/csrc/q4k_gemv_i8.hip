// Q4_K decode GEMV (M = 1..2 activation rows per pass) on the int8 matrix cores of gfx950.
//
// y[n] = sum over super-blocks b of  d_b * sum_s sc_s * (sum_k q_k x_k)  -  dmin_b * sum_s mn_s * (sum_k x_k)
// (s: the 8 sub-blocks of 32 weights, q: 4-bit quants, sc/mn: 6-bit scale and min, d/dmin: f16).
//
// The inner sums  sum_k q_k x_k  are exact integer dot products: the activations of one
// super-block column (256 values) are quantised ONCE per launch to 21-bit integers
// X = round(x * 2^E) (E from the column's largest magnitude) and split into three signed
// 7-bit digits X = x0 * 2^14 + x1 * 2^7 + x2, each a valid int8.  v_mfma_i32_16x16x64_i8 then
// multiplies 16 weight rows x 64 weights (two sub-blocks) by up to 16 "activation columns":
// the three digits of four sub-blocks occupy 12 of them, so a pair of MFMAs leaves, in lane
// (row j, group g), the three digit sums of sub-block g of weight row j.  The nibbles only need
// `& 0x0F0F0F0F` / `>> 4 & 0x0F0F0F0F` to become int8 operands (3 vector ops per 8 weights),
// the 6-bit scales are applied to the integer sums with 24-bit integer multiply-adds, and one
// int->float conversion per digit and super-block brings in d, dmin and 2^-E.  The result
// carries every activation to 2^-21 of its column's maximum and is otherwise exact up to the
// final f32 roundings (observed 1e-6 relative L2 against an f64 evaluation).
//
// Work split: a workgroup is 16 waves; wave w owns super-block columns w, w+16, ... of every
// weight row the workgroup visits, so the activation operands of a wave never change: they
// are built once (each wave loads, quantises and lays out its own columns, no workgroup
// barrier) and stay in registers.  A work unit is 16 weight rows x one super-block = 2304
// contiguous-per-row bytes, fetched by the load unit straight into the wave's private LDS
// ring (global_load_lds, 16 bytes per lane, 9 lanes per row) with up to `depth` units in
// flight per wave; the wave waits on its own load counter only.  Waves meet once per 16-row
// tile, without waiting: each leaves its K-slice partial sums in LDS and bumps a counter, the
// wave that arrives last adds them in wave order (deterministic) and writes the outputs.
#include <algorithm>
#include <cstdlib>

#include "dh_common.h"
#include "q4k_device.h"

namespace {

using dh::kBlockBytes;
using dh::kQK;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

constexpr int kWaves = 16;
constexpr int kTileRows = 16;
constexpr int kStage = kTileRows * kBlockBytes;   // 2304 bytes per ring stage
constexpr int kUnitLoads = 3;                     // ceil(16 rows * 9 pieces / 64 lanes)
constexpr int kSlots = 4;                         // tiles a fast wave may run ahead of the slowest
constexpr int kMaxDepth = 5;
constexpr size_t kMaxLds = 160 * 1024;

#define DH_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
// s_waitcnt with only the vector-memory counter set (6 bits, split 4 + 2 in the encoding).
#define DH_WAIT_VM(k) __builtin_amdgcn_s_waitcnt(((k) & 0xF) | (((k) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

// Waits until at most n of this wave's vector-memory loads are outstanding (loads complete in
// issue order).  Counts without a case wait for everything, which is always safe.
__device__ __forceinline__ void wait_vm_at_most(int n) {
  switch (n) {
    case 3: DH_WAIT_VM(3); break;
    case 6: DH_WAIT_VM(6); break;
    case 9: DH_WAIT_VM(9); break;
    case 12: DH_WAIT_VM(12); break;
    case 15: DH_WAIT_VM(15); break;
    default: DH_WAIT_VM(0); break;
  }
}

struct I8Args {
  const float* A;        // [M][K]
  const uint8_t* W;      // Q4_K rows
  const uint8_t* W2;     // second matrix (DUAL) or null
  void* C;               // [M][N] f32 or f16
  const float* residual; // [M][N] or null
  int M, N, K, nb;
  int depth;             // ring stages per wave
  int gsize, ngroups;    // waves per group (= min(nb, 16)) and groups per workgroup
  int group_mul;         // ceil(65536 / gsize): wave / gsize = wave * group_mul >> 16 for wave < 16
  int tiles_base, tiles_rem;   // 16-row tiles per group: floor and remainder of tiles / (grid * ngroups)
  float alpha;
  int c_f16, activation;
  float clamp_max;
  const float* norm_weight;   // RMSNorm prologue (null = off)
  float norm_eps;
  int norm_weight_offset;
};

// Largest value across the wave, wave-uniform (DPP inside the 16-lane rows, then scalar).
__device__ __forceinline__ float wave_max_uniform(float v) {
  auto shr = [](float x, auto ctrl) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(x), __float_as_int(x), decltype(ctrl)::value, 0xF, 0xF, false));
  };
  v = fmaxf(v, shr(v, std::integral_constant<int, 0x111>{}));
  v = fmaxf(v, shr(v, std::integral_constant<int, 0x112>{}));
  v = fmaxf(v, shr(v, std::integral_constant<int, 0x114>{}));
  v = fmaxf(v, shr(v, std::integral_constant<int, 0x118>{}));
  const int b = __float_as_int(v);
  return fmaxf(fmaxf(__int_as_float(__builtin_amdgcn_readlane(b, 15)), __int_as_float(__builtin_amdgcn_readlane(b, 31))),
               fmaxf(__int_as_float(__builtin_amdgcn_readlane(b, 47)), __int_as_float(__builtin_amdgcn_readlane(b, 63))));
}

// Sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48, left in all of them.
__device__ __forceinline__ float sum_lane_groups(float v) {
  const uint32_t u = __float_as_uint(v);
  auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const uint32_t w = __float_as_uint(v);
  auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Sum over aligned groups of 8 lanes, left in all of them.
__device__ __forceinline__ int sum8_i32(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false);    // quad_perm [1,0,3,2]
  v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, false);    // quad_perm [2,3,0,1]
  v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, false);   // row_half_mirror
  return v;
}

#ifdef DH_I8_TRACE
__device__ unsigned long long dh_i8_trace[256 * 16 * 32];
#define DH_TS(k) do { if (lane == 0) ts_lds[wave][(k) & 31] = wall_clock64(); } while (0)
#else
#define DH_TS(k) do {} while (0)
#endif

template <int MT, bool DUAL, int NCOL, bool VEC>
__global__ __launch_bounds__(64 * kWaves, 1) void q4k_gemv_i8_kernel(const I8Args a) {
  constexpr int NMAT = DUAL ? 2 : 1;
#ifdef DH_I8_TRACE
  __shared__ unsigned long long ts_lds[kWaves][32];
#endif
  __shared__ float red[kSlots][kWaves][NMAT][MT][16];       // K-slice partial sums per tile slot
  __shared__ unsigned done[kSlots][kWaves];                 // [slot][group]: waves that delivered
  __shared__ float norm_ss[kWaves][MT];
  __shared__ __align__(16) unsigned char xst[kWaves][800];  // per wave: three digit planes of one column + 8 sums
  extern __shared__ __align__(16) unsigned char ring[];     // [kWaves][depth][kStage]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
#ifdef DH_I8_TRACE
  if (lane < 32) ts_lds[wave][lane] = 0ull;
#endif
  DH_TS(0);
  // Every kernel argument is fetched in one batch here (left alone the compiler fetches some of
  // them only where they are first used: a second, dependent trip to memory).
  asm volatile("" :: "s"(a.A), "s"(a.W), "s"(a.W2), "s"(a.C), "s"(a.residual), "s"(a.norm_weight));
  asm volatile("" :: "s"(a.M), "s"(a.N), "s"(a.K), "s"(a.nb), "s"(a.depth), "s"(a.gsize), "s"(a.ngroups),
               "s"(a.group_mul), "s"(a.tiles_base), "s"(a.tiles_rem), "s"(a.c_f16), "s"(a.activation),
               "s"(a.norm_weight_offset));
  asm volatile("" :: "s"(a.alpha), "s"(a.clamp_max), "s"(a.norm_eps));
  // The arrival counters are zeroed and the workgroup meets before anything else: at this point
  // the barrier costs only the skew of the wave launches.
  if (tid < kSlots * kWaves) (&done[0][0])[tid] = 0u;
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  const int group = (wave * a.group_mul) >> 16, col0 = wave - group * a.gsize;     // wave / gsize
  const bool idle = group >= a.ngroups;
  if (idle) return;

  const int D = a.depth;
  const int64_t row_bytes = (int64_t)a.nb * kBlockBytes;
  const int ngr_total = (int)gridDim.x * a.ngroups;
  const int gid = (int)blockIdx.x * a.ngroups + group;
  // tiles gid, gid + ngr_total, ...: tiles_base of them, one more for the first tiles_rem groups
  const int ntl = a.tiles_base + (gid < a.tiles_rem ? 1 : 0);
  const int ntl_max = a.tiles_base + (a.tiles_rem > 0 ? 1 : 0);               // the same in every wave
  const int bpw = a.gsize == kWaves ? (a.nb - col0 + kWaves - 1) >> 4 : 1;
  unsigned char* my_ring = ring + (size_t)wave * D * kStage;
  const bool norm = a.norm_weight != nullptr;

  // piece p = t*64 + lane of a unit: row p/9, 16-byte piece p%9 of that row's super-block
  uint32_t goff[kUnitLoads];
#pragma unroll
  for (int t = 0; t < kUnitLoads; t++) {
    const int p = t * 64 + lane, r = p / 9;
    goff[t] = p < 9 * kTileRows ? (uint32_t)(r * row_bytes + (p - r * 9) * 16) : 0xFFFFFFFFu;
  }

  struct { int tl, mat, i; } ic = {0, 0, 0};
  int issue_stage = 0, issued = 0;
#define DH_ISSUE_NEXT()                                                                           \
  do {                                                                                            \
    if (ic.tl < ntl) {                                                                            \
      const int tile_ = gid + ic.tl * ngr_total;                                                  \
      const uint8_t* base_ = ((DUAL && ic.mat) ? a.W2 : a.W) + (int64_t)tile_ * kTileRows * row_bytes + \
                             (int64_t)(col0 + kWaves * ic.i) * kBlockBytes;                       \
      unsigned char* st_ = my_ring + issue_stage * kStage;                                        \
      const int rows_left_ = a.N - tile_ * kTileRows;                                             \
      if (rows_left_ >= kTileRows) {                                                              \
        _Pragma("unroll") for (int t = 0; t < kUnitLoads; t++) {                                  \
          if (goff[t] != 0xFFFFFFFFu)                                                             \
            __builtin_amdgcn_global_load_lds(base_ + goff[t], DH_LDS_PTR(st_ + t * 1024), 16, 0, 0); \
        }                                                                                         \
      } else {                                                                                    \
        _Pragma("unroll") for (int t = 0; t < kUnitLoads; t++) {                                  \
          const int p_ = t * 64 + lane, r_ = p_ / 9;                                              \
          const int64_t o_ = (int64_t)min(r_, rows_left_ - 1) * row_bytes + (p_ - r_ * 9) * 16;   \
          if (goff[t] != 0xFFFFFFFFu)                                                             \
            __builtin_amdgcn_global_load_lds(base_ + o_, DH_LDS_PTR(st_ + t * 1024), 16, 0, 0);   \
        }                                                                                         \
      }                                                                                           \
      issued++;                                                                                   \
      issue_stage = issue_stage + 1 == D ? 0 : issue_stage + 1;                                   \
      if (++ic.i == bpw) {                                                                        \
        ic.i = 0;                                                                                 \
        if (++ic.mat == NMAT) { ic.mat = 0; ic.tl++; }                                            \
      }                                                                                           \
    }                                                                                             \
  } while (0)

  // ---- 1. this wave's activation columns: lane t holds elements 4t .. 4t+3 of each column.
  // Fast path (K a multiple of 4, 16-byte aligned rows): the loads are hand-issued so that the
  // ring can be put in flight behind them and only THEY are waited for.
  v4f xr[NCOL][MT], wr[NCOL];
#pragma unroll
  for (int i = 0; i < NCOL; i++) {
    const int k0 = (col0 + kWaves * i) * kQK + 4 * lane;
    const bool in = i < bpw && k0 < a.K;
    if constexpr (VEC) {
#pragma unroll
      for (int m = 0; m < MT; m++) {
        const float* p = a.A + (int64_t)min(m, a.M - 1) * a.K + (in ? k0 : 0);
        asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(xr[i][m]) : "v"(p) : "memory");
      }
      if (norm) {
        const float* p = a.norm_weight + (in ? k0 : 0);
        asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(wr[i]) : "v"(p) : "memory");
      }
    } else {
#pragma unroll
      for (int m = 0; m < MT; m++) {
#pragma unroll
        for (int e = 0; e < 4; e++)
          xr[i][m][e] = (in && k0 + e < a.K) ? a.A[(int64_t)min(m, a.M - 1) * a.K + k0 + e] : 0.f;
      }
#pragma unroll
      for (int e = 0; e < 4; e++) wr[i][e] = (norm && in && k0 + e < a.K) ? a.norm_weight[k0 + e] : 0.f;
    }
  }
  if constexpr (!VEC) DH_WAIT_VM(0);
  DH_TS(1);

  // ---- 2. first ring stage only: a wave stalls while it issues loads into a full memory pipeline,
  // and nothing of what follows needs more than the first unit
  DH_ISSUE_NEXT();
  DH_TS(2);

  // ---- 3. wait for the activations only (the ring loads were issued after them)
  if constexpr (VEC) {
    wait_vm_at_most(issued * kUnitLoads);
#pragma unroll
    for (int i = 0; i < NCOL; i++) {
#pragma unroll
      for (int m = 0; m < MT; m++) asm volatile("" : "+v"(xr[i][m]));
      if (norm) asm volatile("" : "+v"(wr[i]));
    }
  }

  DH_TS(3);
  // ---- 4. quantise and lay out the A operands
  // MFMA pair cc (sub-blocks 4cc .. 4cc+3), half ab: lane (i = lane & 15, kg = lane >> 4) supplies
  // operand row i = 4g + digit for k-slots of lane group kg, which hold bytes 16(kg&1) + 8ab + 0..7
  // of chunk 2cc + (kg >> 1): low nibbles (sub-block g even) in operand bytes 0..7, high nibbles (g
  // odd) in bytes 8..15.  Rows of another chunk's sub-blocks, and the fourth row of every group, are 0.
  v4i aop[NCOL][MT][2][2];
  float sxa[NCOL][MT], sxb[NCOL][MT], xinv[NCOL][MT];
  const int kg = lane >> 4;
  {
    const int irow = lane & 15, g = irow >> 2, dg = irow & 3;
    const bool active = dg < 3 && (g >> 1) == (kg >> 1);
    unsigned char* st = xst[wave];
    const uint32_t st_lds = (uint32_t)(uintptr_t)DH_LDS_PTR(st);
    float ss[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) ss[m] = 0.f;
#pragma unroll
    for (int i = 0; i < NCOL; i++) {
      const int k0 = (col0 + kWaves * i) * kQK + 4 * lane;
      const bool in = i < bpw && k0 < a.K;
#pragma unroll
      for (int m = 0; m < MT; m++) {
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          v[e] = (in && m < a.M) ? xr[i][m][e] : 0.f;
          if (norm) {
            ss[m] = fmaf(v[e], v[e], ss[m]);
            v[e] *= a.norm_weight_offset ? 1.0f + wr[i][e] : wr[i][e];
          }
        }
        const float mx = wave_max_uniform(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
        int ex = (int)((__float_as_uint(mx) >> 23) & 0xFF) - 127;     // mx < 2^(ex+1)
        ex = max(-100, min(100, ex));
        if (mx == 0.f) ex = 0;
        const float sf = __uint_as_float((uint32_t)(127 + 19 - ex) << 23);   // |x| * sf < 2^20
        xinv[i][m] = __uint_as_float((uint32_t)(127 - 19 + ex) << 23);
        // X = round(x * sf) sits in the low mantissa bits of x * sf + 1.5 * 2^23 (two's complement)
        uint32_t b[4], d2[4], d1[4], d0[4];
        uint32_t xs = 0u;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          b[e] = __float_as_uint(fmaf(v[e], sf, 12582912.0f));
          xs += b[e];
          d2[e] = (uint32_t)__builtin_amdgcn_sbfe((int)b[e], 0, 7);              // signed low 7 bits
          d1[e] = (uint32_t)__builtin_amdgcn_sbfe((int)(b[e] + 64u), 7, 7);
          d0[e] = (b[e] + 8256u) >> 14;                                          // byte 0 = top digit
        }
        const uint32_t lo01 = 0x0c0c0400u, hi23 = 0x04000c0cu;   // byte 0 of (src1, src0) -> bytes 0,1 / 2,3
        const uint32_t pk0 = __builtin_amdgcn_perm(d0[1], d0[0], lo01) | __builtin_amdgcn_perm(d0[3], d0[2], hi23);
        const uint32_t pk1 = __builtin_amdgcn_perm(d1[1], d1[0], lo01) | __builtin_amdgcn_perm(d1[3], d1[2], hi23);
        const uint32_t pk2 = __builtin_amdgcn_perm(d2[1], d2[0], lo01) | __builtin_amdgcn_perm(d2[3], d2[2], hi23);
        // sum of the quantised activations of each sub-block (8 lanes x 4 elements)
        const float sxf = (float)sum8_i32((int)(xs - 4u * 0x4B400000u)) * xinv[i][m];
        // lane L wrote the digit bytes of elements 4L .. 4L+3 of plane `digit`; an operand lane
        // reads the eight bytes its k-slots cover
        reinterpret_cast<uint32_t*>(st)[lane] = pk0;
        reinterpret_cast<uint32_t*>(st)[64 + lane] = pk1;
        reinterpret_cast<uint32_t*>(st)[128 + lane] = pk2;
        if ((lane & 7) == 0) reinterpret_cast<float*>(st)[192 + (lane >> 3)] = sxf;
        // (hand-written reads: the compiler would wait for the weight loads in flight before
        // any LDS read of its own, because those loads write LDS too.  LDS executes a wave's
        // operations in order, so the stores above are seen.)
        uint2 t00, t01, t10, t11;
        float s_a, s_b;
        asm volatile(
            "ds_read_b64 %0, %6\n\t"
            "ds_read_b64 %1, %6 offset:8\n\t"
            "ds_read_b64 %2, %6 offset:128\n\t"
            "ds_read_b64 %3, %6 offset:136\n\t"
            "ds_read_b32 %4, %7 offset:768\n\t"
            "ds_read_b32 %5, %7 offset:784\n\t"
            "s_waitcnt lgkmcnt(0)"
            : "=&v"(t00), "=&v"(t01), "=&v"(t10), "=&v"(t11), "=&v"(s_a), "=&v"(s_b)
            : "v"(st_lds + 256 * min(dg, 2) + 32 * g + 16 * (kg & 1)), "v"(st_lds + 4 * kg)
            : "memory");
        const uint2 tt[2][2] = {{t00, t01}, {t10, t11}};
#pragma unroll
        for (int cc = 0; cc < 2; cc++) {
#pragma unroll
          for (int ab = 0; ab < 2; ab++) {
            const int t0 = active ? (int)tt[cc][ab].x : 0, t1 = active ? (int)tt[cc][ab].y : 0;
            aop[i][m][cc][ab] = (g & 1) ? v4i{0, 0, t0, t1} : v4i{t0, t1, 0, 0};
          }
        }
        sxa[i][m] = s_a;
        sxb[i][m] = s_b;
      }
    }
    if (norm) {
#pragma unroll
      for (int m = 0; m < MT; m++) {
        const float t = dh::wave_sum_uniform(ss[m]);
        if (lane == 0) norm_ss[wave][m] = t;
      }
    }
  }

  for (int d = 1; d < D; d++) DH_ISSUE_NEXT();
  DH_TS(4);
  // ---- 5. stream the units
  const int j = lane & 15;
  // LDS byte address of this lane's header inside stage 0, and of its 16 nibble bytes of chunk
  // (kg >> 1) (chunk 2 + (kg >> 1) is 64 bytes further)
  const uint32_t lane_hdr = (uint32_t)(uintptr_t)DH_LDS_PTR(my_ring) + (uint32_t)j * kBlockBytes;
  const uint32_t lane_q = lane_hdr + 16 + 32 * (kg >> 1) + 16 * (kg & 1);
  const uint32_t sh_lo = 8 * kg;           // bit offset of this lane's byte in the header words

  int consumed = 0, cstage = 0;
#pragma unroll 1
  for (int tl = 0; tl < ntl_max; tl++) {
    const int slot = tl % kSlots;
    if (tl < ntl) {
      const int tile = gid + tl * ngr_total;
#pragma unroll 1
      for (int mat = 0; mat < NMAT; mat++) {
        float acc[MT];
#pragma unroll
        for (int m = 0; m < MT; m++) acc[m] = 0.f;
#pragma unroll
        for (int i = 0; i < NCOL; i++) {
          if (i < bpw) {
            wait_vm_at_most((issued - consumed - 1) * kUnitLoads);
            DH_TS(5 + consumed);
            const uint32_t hp = lane_hdr + cstage * kStage, qp = lane_q + cstage * kStage;
            v4u h, q0, q1;
            asm volatile(
                "ds_read_b128 %0, %3\n\t"
                "ds_read_b128 %1, %4\n\t"
                "ds_read_b128 %2, %4 offset:64\n\t"
                "s_waitcnt lgkmcnt(0)"
                : "=&v"(h), "=&v"(q0), "=&v"(q1)
                : "v"(hp), "v"(qp)
                : "memory");
            consumed++;
            cstage = cstage + 1 == D ? 0 : cstage + 1;
            DH_ISSUE_NEXT();            // the stage just read is free again
            // 6-bit scales and mins of sub-blocks kg and 4 + kg of this lane's weight row
            const int sc_a = (int)((h.y >> sh_lo) & 63u);
            const int sc_b = (int)(((h.w >> sh_lo) & 15u) | (((h.y >> (sh_lo + 6)) & 3u) << 4));
            const float mn_a = (float)((h.z >> sh_lo) & 63u);
            const float mn_b = (float)(((h.w >> (sh_lo + 4)) & 15u) | (((h.z >> (sh_lo + 6)) & 3u) << 4));
            const float d = f16lo(h.x), dmin = f16hi(h.x);
            v4i dd[2][MT];
#pragma unroll
            for (int cc = 0; cc < 2; cc++) {
              const v4u q = cc ? q1 : q0;
              const v4i ba = {(int)(q.x & 0x0F0F0F0Fu), (int)(q.y & 0x0F0F0F0Fu),
                              (int)((q.x >> 4) & 0x0F0F0F0Fu), (int)((q.y >> 4) & 0x0F0F0F0Fu)};
              const v4i bb = {(int)(q.z & 0x0F0F0F0Fu), (int)(q.w & 0x0F0F0F0Fu),
                              (int)((q.z >> 4) & 0x0F0F0F0Fu), (int)((q.w >> 4) & 0x0F0F0F0Fu)};
#pragma unroll
              for (int m = 0; m < MT; m++) {
                v4i t = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[i][m][cc][0], ba, v4i{0, 0, 0, 0}, 0, 0, 0);
                dd[cc][m] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[i][m][cc][1], bb, t, 0, 0, 0);
              }
            }
#pragma unroll
            for (int m = 0; m < MT; m++) {
              // |digit sum| <= 32*15*64 and the scale is 6 bits: 24-bit multiplies are exact
              const int p0 = __mul24(sc_a, dd[0][m][0]) + __mul24(sc_b, dd[1][m][0]);
              const int p1 = __mul24(sc_a, dd[0][m][1]) + __mul24(sc_b, dd[1][m][1]);
              const int p2 = __mul24(sc_a, dd[0][m][2]) + __mul24(sc_b, dd[1][m][2]);
              const float t = fmaf((float)p0, 16384.f, fmaf((float)p1, 128.f, (float)p2));
              const float mins = fmaf(mn_a, sxa[i][m], mn_b * sxb[i][m]);
              acc[m] = fmaf(d * xinv[i][m], t, fmaf(-dmin, mins, acc[m]));
            }
          }
        }
        // the four lane groups hold different sub-blocks of the same 16 rows
#pragma unroll
        for (int m = 0; m < MT; m++) {
          const float s = sum_lane_groups(acc[m]);
          if (lane < 16) red[slot][wave][mat][m][lane] = s;
        }
      }
      // ---- tile end.  Nobody waits: each wave reports its partial sums and moves on; the wave of
      // the group that arrives last adds the K slices in wave order and writes the outputs.  LDS
      // executes a wave's operations in order, so every earlier arrival's partials are in place.
      // (Hand-written LDS atomic: the compiler would put a wait for all loads in flight in front
      // of its own, because the ring loads write LDS too.)
      unsigned arrived = 0;
      if (lane == 0) {
        const uint32_t cnt_addr = (uint32_t)(uintptr_t)DH_LDS_PTR(&done[slot][group]);
        asm volatile("ds_add_rtn_u32 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(arrived) : "v"(cnt_addr), "v"(1u) : "memory");
      }
      arrived = __builtin_amdgcn_readfirstlane(arrived);
      asm volatile("" ::: "memory");
      if ((int)arrived == a.gsize - 1) {
        const int64_t row = (int64_t)tile * kTileRows + j;
        const int w0 = group * a.gsize;
#pragma unroll 1
        for (int m = kg; m < MT; m += 4) {
          if (m < a.M && row < a.N) {
            float sg = 0.f, su = 0.f;
            for (int w = 0; w < a.gsize; w++) {
              sg += red[slot][w0 + w][0][m][j];
              if (DUAL) su += red[slot][w0 + w][NMAT - 1][m][j];
            }
            if (norm) {
              float tot = 0.f;
              for (int w = 0; w < a.gsize; w++) tot += norm_ss[w0 + w][m];
              const float inv = 1.0f / sqrtf(tot / (float)a.K + a.norm_eps);
              sg *= inv;
              su *= inv;
            }
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
        if (lane == 0) done[slot][group] = 0u;
      }
    }
    DH_TS(20 + tl);
    // more tiles than slots: keep the waves within one tile of each other instead
    if (ntl_max > kSlots) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  }
  DH_TS(31);
#ifdef DH_I8_TRACE
  if (lane < 32 && blockIdx.x < 256) dh_i8_trace[(blockIdx.x * 16 + wave) * 32 + lane] = ts_lds[wave][lane];
#endif
#undef DH_ISSUE_NEXT
}

int env_int(const char* name, int dflt) {
  const char* e = getenv(name);
  return e ? atoi(e) : dflt;
}

template <int MT, bool DUAL, int NCOL, bool VEC>
int launch_i8_vec(I8Args a, const char* op) {
  constexpr int NMAT = DUAL ? 2 : 1;
  auto kern = q4k_gemv_i8_kernel<MT, DUAL, NCOL, VEC>;
  const size_t fixed = sizeof(float) * kSlots * kWaves * NMAT * MT * 16 + sizeof(unsigned) * kSlots * kWaves +
                       sizeof(float) * kWaves * MT + (size_t)kWaves * 800 + 256
#ifdef DH_I8_TRACE
                       + 4096
#endif
      ;
  static bool attr_set = false;   // once per instantiation: the call costs microseconds
  if (!attr_set) {
    DH_CHECK_HIP(op, hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)(kMaxLds - fixed)));
    attr_set = true;
  }
  static const int env_depth = env_int("DH_GEMV_DEPTH", 0);
  const int ncu = dh::num_cus();
  a.gsize = std::min(a.nb, kWaves);
  a.ngroups = kWaves / a.gsize;
  const int64_t ntiles = dh::ceil_div(a.N, kTileRows);
  const int grid = (int)std::min<int64_t>(dh::ceil_div(ntiles, a.ngroups), ncu);
  // units one wave streams: no point in more ring stages than that
  const int64_t tiles_per_group = dh::ceil_div(ntiles, (int64_t)grid * a.ngroups);
  a.group_mul = (65536 + a.gsize - 1) / a.gsize;
  a.tiles_base = (int)(ntiles / ((int64_t)grid * a.ngroups));
  a.tiles_rem = (int)(ntiles % ((int64_t)grid * a.ngroups));
  const int bpw = a.gsize == kWaves ? (int)dh::ceil_div(a.nb, kWaves) : 1;
  int depth = (int)std::min<int64_t>(kMaxDepth, tiles_per_group * NMAT * bpw);
  while (depth > 1 && fixed + (size_t)kWaves * depth * kStage > kMaxLds) depth--;
  if (env_depth > 0) depth = std::min(depth, env_depth);
  a.depth = depth;
  const size_t dyn = (size_t)kWaves * depth * kStage;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * kWaves), dyn, dh::stream(), a);
  DH_CHECK_LAUNCH(op);
  return 0;
}

// Fast path: K a multiple of 4 and 16-byte aligned rows (vector loads of the activations).
template <int MT, bool DUAL, int NCOL>
int launch_i8(const I8Args& a, const char* op) {
  const bool vec = (a.K & 3) == 0 && (reinterpret_cast<uintptr_t>(a.A) & 15) == 0 &&
                   (!a.norm_weight || (reinterpret_cast<uintptr_t>(a.norm_weight) & 15) == 0);
  return vec ? launch_i8_vec<MT, DUAL, NCOL, true>(a, op) : launch_i8_vec<MT, DUAL, NCOL, false>(a, op);
}

template <bool DUAL>
int dispatch_i8(const I8Args& a, const char* op) {
  const int ncol = a.nb >= kWaves ? (int)dh::ceil_div(a.nb, kWaves) : 1;
  if (a.M == 1) {
    if (ncol == 1) return launch_i8<1, DUAL, 1>(a, op);
    if (ncol == 2) return launch_i8<1, DUAL, 2>(a, op);
    if (ncol == 3) return launch_i8<1, DUAL, 3>(a, op);
  } else if (a.M == 2) {
    if (ncol == 1) return launch_i8<2, DUAL, 1>(a, op);
  }
  return -1;
}

}  // namespace

#ifdef DH_I8_TRACE
extern "C" int dh_debug_i8_trace(void* host_dst) {
  return (int)hipMemcpyFromSymbol(host_dst, HIP_SYMBOL(dh_i8_trace), sizeof(dh_i8_trace));
}
#endif

namespace dh {

int q4k_gemv_i8(const char* op, const float* A, const uint8_t* W, const uint8_t* W2, void* C, int c_f16,
                const float* residual, int M, int N, int K, float alpha, int activation, float clamp_max,
                const float* norm_weight, float norm_eps, int norm_weight_offset) {
  static const int off = env_int("DH_GEMV_I8_OFF", 0);
  if (off || M < 1 || M > 2) return -1;
  // the unit offsets are 32-bit: 15 rows of a tile must stay below 4 GB (any realistic K does)
  I8Args a{};
  a.A = A; a.W = W; a.W2 = W2; a.C = C; a.residual = residual;
  a.M = M; a.N = N; a.K = K; a.nb = (K + kQK - 1) / kQK;
  a.alpha = alpha; a.c_f16 = c_f16; a.activation = activation; a.clamp_max = clamp_max;
  a.norm_weight = norm_weight; a.norm_eps = norm_eps; a.norm_weight_offset = norm_weight_offset;
  return W2 ? dispatch_i8<true>(a, op) : dispatch_i8<false>(a, op);
}

}  // namespace dh
