// Q4_K decode GEMV (M = 1..2 activation rows per pass) on the int8 matrix cores of gfx950.
//
// y[n] = sum over super-blocks b of  d_b * sum_s sc_s * (sum_k q_k x_k)  -  dmin_b * sum_s mn_s * (sum_k x_k)
// (s: the 8 sub-blocks of 32 weights, q: 4-bit quants, sc/mn: 6-bit scale and min, d/dmin: f16).
//
// The inner sums  sum_k q_k x_k  are exact integer dot products: the activations of one
// super-block column (256 values) are quantised ONCE per launch to 21-bit integers
// X = round(x * 2^E) (E from the largest magnitude of each 32-element sub-block) and split into three
// 7-bit digits X = x0 * 2^14 + x1 * 2^7 + x2 (x0 signed, x1 and x2 0..127), each a valid int8.
// v_mfma_i32_16x16x64_i8 then multiplies 16 weight rows x 64 weights by up to 16 "activation rows":
// the three digits of four sub-blocks occupy 12 of them, so a pair of MFMAs leaves, in lane (weight
// row j, group g), the three digit sums of sub-block g of weight row j.  The nibbles only need
// `& 0x0F0F0F0F` / `>> 4 & 0x0F0F0F0F` to become int8 operands (3 vector ops per 8 weights), the
// three digit sums are put together as integers (that IS sum_k q_k X_k, exactly), and one int->float
// conversion per sub-block brings in the scale, d, dmin and 2^-E.  The result carries every
// activation to 2^-20 of its sub-block's maximum and is otherwise exact up to the final f32
// roundings (observed 1e-6 relative L2 against an f64 evaluation).
//
// Work split: a workgroup of 16 waves owns 16-row tiles; a work unit is 16 weight rows x one
// super-block column = 2304 bytes (144 contiguous per row).  Units are NOT bound to waves: every
// wave draws the next unit of the workgroup from a counter in LDS, has the load unit fetch it
// straight into its private LDS ring (global_load_lds, 16 bytes per lane, 9 lanes per row), and
// reads the activation operands of the unit's column from LDS.  Those are prepared once per
// launch: wave w quantises columns w, w+16, .. and raises a flag per column, with its first
// weight unit already in flight; a wave that meets a column whose flag is not up yet waits for it.  Waves that get the memory pipeline first (the hardware favours the
// oldest) simply draw more units, so all sixteen finish together and the pipeline stays full until
// the end.  A unit's 16 partial sums go to LDS; the wave that delivers the last unit of a tile
// adds them in column order (deterministic) and writes the outputs.  The only workgroup barrier
// is one at the very start.
#include <algorithm>
#include <cstdlib>
#include <type_traits>

#include "dh_common.h"
#include "q4k_device.h"
#include "q4k_i8_device.h"

namespace {

using dh::kBlockBytes;
using dh::kQK;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef uint32_t v2u __attribute__((ext_vector_type(2)));

constexpr int kWaves = 16;
constexpr int kTileRows = 16;
constexpr int kStage = 3 * 1024;                   // a ring stage: one unit (16 rows x 144 bytes = 2304) as three full
                                                   // 64-lane loads of 16 bytes: the third one's lanes past the unit land in
                                                   // the stage's own tail, so no load needs a lane mask
constexpr int kUnitLoads = 3;                     // load instructions of a full unit: ceil(16 rows * 9 pieces / 64 lanes)
constexpr int kMaxDepth = 1;                      // ring stages per wave (2..5 measured slower: the queue already keeps 16 units in flight)
constexpr int kSlotDepth = 3;                     // what the tile-slot count is sized for
constexpr int kMaxSlots = 32;                     // tiles whose partial sums may be in LDS at once
constexpr int kZeroBytes = 144;                   // what a lane without an operand reads
constexpr size_t kMaxLds = 160 * 1024;
// a finished tile's partial sums are read four columns at a time: the last read of the last slot reaches
// up to twelve columns (of 64 bytes per activation row) past it, into the counters and this padding
constexpr int kReadAhead = 12 * 64;
constexpr int kSpinLimit = 1 << 18;               // polls of a wait inside the workgroup before the wave gives up

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
    case 6: DH_WAIT_VM(6); break;
    default: DH_WAIT_VM(0); break;
  }
}

struct I8Args {
  const float* A;        // [M][K] f32, or f16 in the AF16 kernels (a_f16 set)
  const uint8_t* W;      // Q4_K rows
  const uint8_t* W2;     // second matrix (DUAL) or null
  void* C;               // [M][N] f32 or f16
  const float* residual; // [M][N] or null
  const float* norm_weight;   // RMSNorm prologue (null = off)
  int M, N, K, nb;
  int a_f16;             // the activations are f16 (widened exactly as they are loaded)
  int depth;             // ring stages per wave
  int rows;              // weight rows per tile (<= 16), chosen so that the tiles divide evenly among the workgroups
  int nlw;               // load instructions per unit: ceil(9 * rows / 64)
  int upt;               // units per tile: nb * (DUAL ? 2 : 1)
  int upt_mul;           // ceil(2^24 / upt): u / upt == (u * upt_mul) >> 24 for the unit counts met here
  int grid;              // workgroups launched
  int tiles_base, tiles_rem;   // 16-row tiles per workgroup: floor and remainder of tiles / grid
  int nslots, slot_shift;   // tile slots for partial sums: a power of two, and its log2
  int c_f16, activation, norm_weight_offset;
  float alpha, clamp_max, norm_eps;
  uint32_t* status;      // the library's kernel status word (host memory the device can write)
};

// One LDS word read by hand (the compiler puts a wait for every weight load in flight in front of
// its own LDS reads, because those loads write LDS too).
__device__ __forceinline__ uint32_t lds_read_u32(uint32_t addr) {
  uint32_t v;
  asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(v) : "v"(addr) : "memory");
  return v;
}

// Layout of the dynamic LDS block, in this order:
//   ring   [16 waves][depth][3072]
//   xq     [nb][MT][kRec]: per column and activation row, digit plane p at 256 p (byte e = digit p
//          of element e), the 8 sub-block sums at 768, their factors 2^-E at 800, the column's sum of squares at 832
//   zeros  [144]
//   red    [nslots][upt][MT][16] partial sums of a tile's units
//   ctr    [0] next unit to draw, [1 + s] units delivered to slot s, [1 + nslots + s] tiles completed
//          in slot s, [1 + 2 nslots + c] column c's operands are in place, [1 + 2 nslots + nb] a wave has given up
template <int MT, bool DUAL, bool VEC, bool AF16 = false>
__global__ __launch_bounds__(64 * kWaves, 1) void q4k_gemv_i8_kernel(const I8Args a) {
  constexpr int NMAT = DUAL ? 2 : 1;
  extern __shared__ __align__(16) unsigned char lds[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Every kernel argument is fetched in one batch here (left alone the compiler fetches some of
  // them only where they are first used: a second, dependent trip to memory).
  asm volatile("" :: "s"(a.A), "s"(a.W), "s"(a.W2), "s"(a.C), "s"(a.residual), "s"(a.norm_weight), "s"(a.status));
  asm volatile("" :: "s"(a.M), "s"(a.N), "s"(a.K), "s"(a.nb), "s"(a.depth), "s"(a.rows), "s"(a.nlw), "s"(a.upt), "s"(a.upt_mul),
               "s"(a.grid), "s"(a.tiles_base), "s"(a.tiles_rem), "s"(a.nslots), "s"(a.slot_shift), "s"(a.c_f16), "s"(a.activation),
               "s"(a.norm_weight_offset));
  asm volatile("" :: "s"(a.alpha), "s"(a.clamp_max), "s"(a.norm_eps));

  constexpr int D = kMaxDepth;
  const int nb = a.nb, upt = a.upt, nslots = a.nslots;
  unsigned char* ring = lds;
  unsigned char* xq = ring + (size_t)kWaves * D * kStage;
  unsigned char* zeros = xq + (size_t)nb * MT * kRec;
  float* red = reinterpret_cast<float*>(zeros + kZeroBytes);
  unsigned* ctr = reinterpret_cast<unsigned*>(red + (size_t)nslots * upt * MT * 16);

  // counters, flags, zero area: set before the barrier, which costs only the skew of the wave launches
  for (int i = tid; i < 2 + 2 * nslots + nb; i += 64 * kWaves) ctr[i] = 0u;
  if (tid >= 64 && tid < 64 + kZeroBytes / 4) reinterpret_cast<uint32_t*>(zeros)[tid - 64] = 0u;

  const int64_t row_bytes = (int64_t)nb * kBlockBytes;
  // byte offsets inside a weight matrix fit 32 bits (checked on the host): a unit's address is one
  // 64-bit base plus 32-bit scalar arithmetic
  const uint32_t wg_off = (uint32_t)blockIdx.x * (uint32_t)a.rows * (uint32_t)row_bytes;   // this workgroup's first tile
  const uint32_t tile_stride = (uint32_t)a.grid * (uint32_t)a.rows * (uint32_t)row_bytes;   // to its next tile
  const int rows_left0 = a.N - (int)blockIdx.x * a.rows;        // rows from the first tile's first row to the end
  const int rows_round = a.grid * a.rows;
  // this workgroup's tiles: blockIdx.x, blockIdx.x + grid, ...
  const int ntl = a.tiles_base + ((int)blockIdx.x < a.tiles_rem ? 1 : 0);
  const int total = ntl * upt;                                  // units of this workgroup
  unsigned char* my_ring = ring + (size_t)wave * D * kStage;
  const bool norm = a.norm_weight != nullptr;

  // piece p = t*64 + lane of a unit: row p/9, 16-byte piece p%9 of that row's super-block
  uint32_t goff[kUnitLoads];
#pragma unroll
  for (int t = 0; t < kUnitLoads; t++) {
    const int p = t * 64 + lane, r = p / 9;
    // (lanes past the tile's pieces fetch piece 0 again: their 16 bytes land behind the unit, unread)
    goff[t] = p < 9 * a.rows ? (uint32_t)(r * row_bytes + (p - r * 9) * 16) : 0u;
  }

  // Unit u of the workgroup = (tile ordinal tl, matrix, column): u = (tl * NMAT + mat) * nb + col.
#define DH_DECODE(u_, tl_, mat_, col_)                                  \
  const int tl_ = (int)(((unsigned)(u_) * (unsigned)a.upt_mul) >> 24);  \
  const int r__##tl_ = (u_) - tl_ * upt;                                \
  const int mat_ = (DUAL && r__##tl_ >= nb) ? 1 : 0;                    \
  const int col_ = r__##tl_ - mat_ * nb;

  // Puts the loads of unit u_ in flight into ring stage stage_.
#define DH_ISSUE(u_, stage_)                                                                      \
  do {                                                                                            \
    DH_DECODE(u_, itl_, imat_, icol_)                                                             \
    const uint32_t off_ = wg_off + (uint32_t)itl_ * tile_stride + (uint32_t)icol_ * kBlockBytes;  \
    const uint8_t* base_ = ((DUAL && imat_) ? a.W2 : a.W) + off_;                                 \
    unsigned char* st_ = my_ring + (stage_) * kStage;                                             \
    const int rows_left_ = rows_left0 - itl_ * rows_round;                                        \
    if (rows_left_ >= a.rows) {                                                                   \
      _Pragma("unroll") for (int t = 0; t < kUnitLoads; t++) {                                    \
        /* the offset is made opaque here so that its widening to 64 bits is not hoisted out of the */ \
        /* unit loop: only then does the load take the form scalar base + 32-bit lane offset        */ \
        uint32_t g_ = goff[t];                                                                    \
        asm volatile("" : "+v"(g_));                                                              \
        __builtin_amdgcn_global_load_lds(base_ + g_, DH_LDS_PTR(st_ + t * 1024), 16, 0, 0);       \
      }                                                                                           \
    } else {                                                                                      \
      _Pragma("unroll") for (int t = 0; t < kUnitLoads; t++) {                                    \
        const int p_ = t * 64 + lane, r_ = p_ / 9;                                                \
        const int64_t o_ = (int64_t)min(r_, rows_left_ - 1) * row_bytes + (p_ - r_ * 9) * 16;     \
        __builtin_amdgcn_global_load_lds(base_ + o_, DH_LDS_PTR(st_ + t * 1024), 16, 0, 0);       \
      }                                                                                           \
    }                                                                                             \
  } while (0)

  // ---- 1. every wave prepares the activation operands of columns wave, wave + 16, ..; lane t
  // holds elements 4t .. 4t+3 of a column.  Per (column, row): three digit planes, the sub-block
  // sums, 2^-E and the sum of squares, then the column's flag.  The activation loads go out BEFORE
  // the workgroup barrier and every weight load after it, so the activations are at the head of the
  // compute unit's memory queue.  (Fast path, K a multiple of 4 and 16-byte aligned rows: the loads
  // are hand-issued so that the first weight unit can follow them and only THEY are waited for.)
  const int kg = lane >> 4;
  constexpr int SC = 3;    // columns per pass (all loads of a pass in flight at once)
  const int my_cols = wave < nb ? (nb - wave + kWaves - 1) >> 4 : 0;
  // (f16 activations: the lane's four elements are two registers, widened after the wait)
  using XRaw = std::conditional_t<AF16, v2u, v4f>;
  XRaw xr[SC][MT];
  v4f wr[SC];
#define DH_LOAD_X(c0_)                                                                            \
  do {                                                                                            \
    _Pragma("unroll") for (int i = 0; i < SC; i++) {                                              \
      if ((c0_) + i < my_cols) {                                                                  \
        const int k0 = (wave + kWaves * ((c0_) + i)) * kQK + 4 * lane;                            \
        if constexpr (VEC) {                                                                      \
          const int kc = k0 < a.K ? k0 : 0;                                                       \
          _Pragma("unroll") for (int m = 0; m < MT; m++) {                                        \
            if constexpr (AF16) {                                                                 \
              const uint16_t* p_ = reinterpret_cast<const uint16_t*>(a.A) + (int64_t)min(m, a.M - 1) * a.K + kc; \
              asm volatile("global_load_dwordx2 %0, %1, off" : "=&v"(xr[i][m]) : "v"(p_) : "memory"); \
            } else {                                                                              \
              const float* p_ = a.A + (int64_t)min(m, a.M - 1) * a.K + kc;                        \
              asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(xr[i][m]) : "v"(p_) : "memory"); \
            }                                                                                     \
          }                                                                                       \
          if (norm) {                                                                             \
            const float* p_ = a.norm_weight + kc;                                                 \
            asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(wr[i]) : "v"(p_) : "memory");  \
          }                                                                                       \
        } else {                                                                                  \
          _Pragma("unroll") for (int e = 0; e < 4; e++) {                                         \
            const int kc = min(k0 + e, a.K - 1);                                                  \
            if constexpr (!AF16) {                                                                \
              _Pragma("unroll") for (int m = 0; m < MT; m++)                                      \
                xr[i][m][e] = a.A[(int64_t)min(m, a.M - 1) * a.K + kc];                           \
            }                                                                                     \
            if (norm) wr[i][e] = a.norm_weight[kc];                                               \
          }                                                                                       \
        }                                                                                         \
      }                                                                                           \
    }                                                                                             \
  } while (0)
  // makes the loaded registers depend on the wait in front of it
#define DH_TIE_X()                                                                                \
  do {                                                                                            \
    _Pragma("unroll") for (int i = 0; i < SC; i++) {                                              \
      _Pragma("unroll") for (int m = 0; m < MT; m++) asm volatile("" : "+v"(xr[i][m]));           \
      if (norm) asm volatile("" : "+v"(wr[i]));                                                   \
    }                                                                                             \
  } while (0)
  DH_LOAD_X(0);
  if constexpr (!VEC) {
    DH_WAIT_VM(0);
    DH_TIE_X();
  }
  // counters, flags and the zero area are in place; costs little more than the skew of the wave launches
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

  // Draws the next unit of the workgroup (wave-uniform result).
  const uint32_t ctr_abs = (uint32_t)(uintptr_t)DH_LDS_PTR(ctr);
  const uint32_t abort_addr = ctr_abs + 4 * (1 + 2 * nslots + nb);
  // A wait inside the workgroup ran into its limit: the wave lets its loads land, leaves the code in the
  // library's status word (the host finds it at its next synchronisation), tells the other waves and ends.
  auto give_up = [&](const uint32_t kind) {
    DH_WAIT_VM(0);
    if (lane == 0) {
      __hip_atomic_store(a.status, dh::kstatus_code(kind, 0u, blockIdx.x), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      ctr[1 + 2 * nslots + nb] = 1u;
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_endpgm();          // the wave ends here (no barrier follows in this kernel)
  };
  auto draw = [&]() -> int {
    unsigned v = 0;
    if (lane == 0)
      asm volatile("ds_add_rtn_u32 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)" : "=&v"(v) : "v"(ctr_abs), "v"(1u) : "memory");
    return (int)__builtin_amdgcn_readfirstlane(v);
  };
  // ---- 2. the first unit's loads go out before anything else is waited for
  int u_ring[kMaxDepth];                   // units in the ring stages (>= total: none)
#pragma unroll
  for (int d = 0; d < kMaxDepth; d++) u_ring[d] = 0x7fffffff;
  int inflight = 0;
  u_ring[0] = draw();
  if (u_ring[0] < total) {
    DH_ISSUE(u_ring[0], 0);
    inflight = 1;
  }
  {
#pragma unroll 1
    for (int c0 = 0; c0 < my_cols; c0 += SC) {
      if (c0 > 0) DH_LOAD_X(c0);
      if constexpr (VEC) {
        // only the activations are waited for (the unit's loads were issued behind them)
        if (c0 == 0 && inflight) wait_vm_at_most(a.nlw); else DH_WAIT_VM(0);
        DH_TIE_X();
      }
#pragma unroll
      for (int i = 0; i < SC; i++) {
        if (c0 + i < my_cols) {
          const int col = wave + kWaves * (c0 + i);
#pragma unroll
          for (int m = 0; m < MT; m++) {
            float v[4], ss = 0.f;
#pragma unroll
            for (int e = 0; e < 4; e++) {
              float raw;
              if constexpr (AF16) raw = (e & 1) ? f16hi(xr[i][m][e >> 1]) : f16lo(xr[i][m][e >> 1]);
              else raw = xr[i][m][e];
              v[e] = (m < a.M && col * kQK + 4 * lane + e < a.K) ? raw : 0.f;
              if (norm) {
                ss = fmaf(v[e], v[e], ss);
                v[e] *= a.norm_weight_offset ? 1.0f + wr[i][e] : wr[i][e];
              }
            }
            unsigned char* rec = xq + (size_t)(col * MT + m) * kRec;
            i8_quantise_store(v, rec, lane);
            if (norm) ss = dh::wave_sum_uniform(ss);
            if (lane == 0) reinterpret_cast<float*>(rec)[kRecSsq / 4] = ss;
          }
          // LDS executes a wave's operations in order: whoever sees the flag sees the record
          if (lane == 0) ctr[1 + 2 * nslots + col] = 1u;
        }
      }
    }
  }
#undef DH_LOAD_X
#undef DH_TIE_X

  // ---- 5. stream the units
  // MFMA pair cc (sub-blocks 4cc .. 4cc+3): the first MFMA takes the low nibbles of the 16 bytes
  // lane (j, kg) holds (bytes 16(kg&1) .. +15 of chunk 2cc + (kg >> 1): sub-block g = 2 (kg >> 1)
  // of the four, elements 16(kg&1) .. +15), the second the high nibbles (sub-block g + 1).  On the
  // activation side lane (i = lane & 15, kg) supplies operand row i = 4g + digit for the same k-slots:
  // 16 digit bytes where its row's sub-block is the one those slots hold, zeros elsewhere (and in
  // the fourth row of every group).
  const int j = lane & 15;
  uint32_t a_mul[2], a_off[2];                  // operand address = record * a_mul + a_off (+ 128 cc)
  {
    const int g = j >> 2, dg = j & 3;
    const uint32_t zero_abs = (uint32_t)(uintptr_t)DH_LDS_PTR(zeros);
    const uint32_t data_off = 256 * min(dg, 2) + 32 * g + 16 * (kg & 1);
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const bool has = dg < 3 && (g >> 1) == (kg >> 1) && (g & 1) == h;
      a_mul[h] = has ? 1u : 0u;
      a_off[h] = has ? data_off : zero_abs;
    }
  }
  const uint32_t xq_abs = (uint32_t)(uintptr_t)DH_LDS_PTR(xq);
  const uint32_t red_abs = (uint32_t)(uintptr_t)DH_LDS_PTR(red);
  // LDS byte address of this lane's header inside stage 0, and of its 16 nibble bytes of chunk
  // (kg >> 1) (chunk 2 + (kg >> 1) is 64 bytes further)
  const uint32_t lane_hdr = (uint32_t)(uintptr_t)DH_LDS_PTR(my_ring) + (uint32_t)j * kBlockBytes;
  const uint32_t lane_q = lane_hdr + 16 + 32 * (kg >> 1) + 16 * (kg & 1);
  const uint32_t sh_lo = 8 * kg;           // bit offset of this lane's byte in the header words

  float inv_rms[MT];                       // RMSNorm prologue: filled by the first tile end this wave meets
  bool have_rms = false;
#pragma unroll
  for (int m = 0; m < MT; m++) inv_rms[m] = 1.f;

  for (int d = 1; d < D; d++) {
    if (u_ring[0] >= total) break;
    const int u = draw();
#pragma unroll
    for (int q = 0; q < kMaxDepth; q++) if (q == d) u_ring[q] = u;
    if (u >= total) break;
    DH_ISSUE(u, d);
    inflight++;
  }

  int cstage = 0;
#pragma unroll 1
  for (;;) {
    int cur = u_ring[0];
#pragma unroll
    for (int q = 1; q < kMaxDepth; q++) cur = q == cstage ? u_ring[q] : cur;
    if (cur >= total) break;              // draws only grow: nothing behind this one either
    DH_DECODE(cur, tl, mat, col)
    const int slot = tl & (nslots - 1);
    // draw the unit that will go into this stage once it has been read (the answer is collected
    // with the reads below)
    unsigned nxt = 0;
    if (lane == 0) asm volatile("ds_add_rtn_u32 %0, %1, %2" : "=&v"(nxt) : "v"(ctr_abs), "v"(1u) : "memory");
    if constexpr (D == 1) DH_WAIT_VM(0); else wait_vm_at_most((inflight - 1) * a.nlw);
    const uint32_t hp = lane_hdr + cstage * kStage, qp = lane_q + cstage * kStage;
    const uint32_t rec = xq_abs + (uint32_t)(col * MT) * kRec;
    const uint32_t gen_addr = ctr_abs + 4 * (1 + nslots + slot);
    const uint32_t flag_addr = ctr_abs + 4 * (1 + 2 * nslots + col);
    // activation rows are handled MP at a time (their operands share the registers); the first
    // batch is read together with the weights
    constexpr int MP = MT < 2 ? MT : 2;
    v4u h, q0, q1;
    v4i ax[MP][2][2];
    v2f sx[MP], xinv[MP];     // activation sums and factors of sub-blocks kg and 4 + kg
    uint32_t gen, flag;
    asm volatile(
        "ds_read_b32 %4, %8\n\t"
        "ds_read_b128 %0, %5\n\t"
        "ds_read_b128 %1, %6\n\t"
        "ds_read_b128 %2, %6 offset:64\n\t"
        "ds_read_b32 %3, %7"
        : "=&v"(h), "=&v"(q0), "=&v"(q1), "=&v"(gen), "=&v"(flag)
        : "v"(hp), "v"(qp), "v"(gen_addr), "v"(flag_addr)
        : "memory");
    // the column's operands, read at once on the expectation that its flag is up (it is, except
    // in the first microseconds of a launch); re-read below if it was not
#define DH_READ_OPERANDS(m0_)                                                                     \
    _Pragma("unroll") for (int m = 0; m < MP; m++) {                                              \
      const uint32_t rm = rec + ((m0_) + m) * kRec;                                               \
      const uint32_t pa = rm * a_mul[0] + a_off[0], pb = rm * a_mul[1] + a_off[1], ps = rm + kRecSums + 4 * kg; \
      asm volatile(                                                                               \
          "ds_read_b128 %0, %6\n\t"                                                               \
          "ds_read_b128 %1, %7\n\t"                                                               \
          "ds_read_b128 %2, %6 offset:128\n\t"                                                    \
          "ds_read_b128 %3, %7 offset:128\n\t"                                                    \
          "ds_read2_b32 %4, %8 offset1:4\n\t"                                                     \
          "ds_read2_b32 %5, %8 offset0:8 offset1:12"                                              \
          : "=&v"(ax[m][0][0]), "=&v"(ax[m][0][1]), "=&v"(ax[m][1][0]), "=&v"(ax[m][1][1]), "=&v"(sx[m]), "=&v"(xinv[m]) \
          : "v"(pa), "v"(pb), "v"(ps)                                                             \
          : "memory");                                                                            \
    }
#define DH_TIE_OPERANDS()                                                                         \
    _Pragma("unroll") for (int m = 0; m < MP; m++)                                                \
      asm volatile("" : "+v"(ax[m][0][0]), "+v"(ax[m][0][1]), "+v"(ax[m][1][0]), "+v"(ax[m][1][1]), "+v"(sx[m]), "+v"(xinv[m]))
    DH_READ_OPERANDS(0)
    // everything above has landed (one wait for all of it; the registers are tied to it)
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(h), "+v"(q0), "+v"(q1), "+v"(gen), "+v"(flag), "+v"(nxt) :: "memory");
    DH_TIE_OPERANDS();
    if (__builtin_amdgcn_readfirstlane(flag) == 0u) {
      // bounded: a wave that is not served within the limit reports it and leaves; so do the others
      int spins = 0;
      do {
        __builtin_amdgcn_s_sleep(2);
        flag = lds_read_u32(flag_addr);
        if (++spins > kSpinLimit || __builtin_amdgcn_readfirstlane(lds_read_u32(abort_addr)) != 0u) break;
      } while (__builtin_amdgcn_readfirstlane(flag) == 0u);
      if (__builtin_amdgcn_readfirstlane(flag) == 0u) {
        give_up(DH_KSTATUS_COLUMN_WAIT);
      }
      DH_READ_OPERANDS(0)
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      DH_TIE_OPERANDS();
    }
    // the stage is free again: put the loads of the unit drawn above in flight
    inflight--;
    {
      const int u = (int)__builtin_amdgcn_readfirstlane(nxt);
#pragma unroll
      for (int q = 0; q < kMaxDepth; q++) if (q == cstage) u_ring[q] = u;
      if (u < total) { DH_ISSUE(u, cstage); inflight++; }
    }
    cstage = cstage + 1 == D ? 0 : cstage + 1;

    // 6-bit scales and mins of sub-blocks kg and 4 + kg of this lane's weight row
    const int sc_a = (int)((h.y >> sh_lo) & 63u);
    const int sc_b = (int)(((h.w >> sh_lo) & 15u) | (((h.y >> (sh_lo + 6)) & 3u) << 4));
    const float mn_a = (float)((h.z >> sh_lo) & 63u);
    const float mn_b = (float)(((h.w >> (sh_lo + 4)) & 15u) | (((h.z >> (sh_lo + 6)) & 3u) << 4));
    const float d = f16lo(h.x), dmin = f16hi(h.x);
    v4i blo[2], bhi[2];
#pragma unroll
    for (int cc = 0; cc < 2; cc++) {
      const v4u q = cc ? q1 : q0;
      blo[cc] = v4i{(int)(q.x & 0x0F0F0F0Fu), (int)(q.y & 0x0F0F0F0Fu), (int)(q.z & 0x0F0F0F0Fu),
                    (int)(q.w & 0x0F0F0F0Fu)};
      bhi[cc] = v4i{(int)((q.x >> 4) & 0x0F0F0F0Fu), (int)((q.y >> 4) & 0x0F0F0F0Fu),
                    (int)((q.z >> 4) & 0x0F0F0F0Fu), (int)((q.w >> 4) & 0x0F0F0F0Fu)};
    }
    // wait (never, in practice) until the tile that used this slot nslots tiles ago is written out
    {
      const unsigned want = (unsigned)tl >> a.slot_shift;
      int spins = 0;
      while (__builtin_amdgcn_readfirstlane(gen) != want) {
        __builtin_amdgcn_s_sleep(1);
        gen = lds_read_u32(gen_addr);
        if (++spins > kSpinLimit || __builtin_amdgcn_readfirstlane(lds_read_u32(abort_addr)) != 0u) break;
      }
      if (__builtin_amdgcn_readfirstlane(gen) != want) {
        give_up(DH_KSTATUS_SLOT_WAIT);
      }
    }
#pragma unroll
    for (int m0 = 0; m0 < MT; m0 += MP) {
      if (m0 > 0) {
        DH_READ_OPERANDS(m0)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        DH_TIE_OPERANDS();
      }
#pragma unroll
      for (int m = 0; m < MP; m++) {
        v4i dd[2];
#pragma unroll
        for (int cc = 0; cc < 2; cc++) {
          v4i t = __builtin_amdgcn_mfma_i32_16x16x64_i8(ax[m][cc][0], blo[cc], v4i{0, 0, 0, 0}, 0, 0, 0);
          dd[cc] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ax[m][cc][1], bhi[cc], t, 0, 0, 0);
        }
        // the four lane groups hold different sub-blocks of the same 16 rows
        const float sres = sum_lane_groups(i8_unit_term(dd[0], dd[1], sc_a, sc_b, mn_a, mn_b, d, dmin, sx[m], xinv[m]));
        if (lane < 16) red[(((size_t)slot * upt + (mat * nb + col)) * MT + m0 + m) * 16 + lane] = sres;
      }
    }
#undef DH_READ_OPERANDS
#undef DH_TIE_OPERANDS
    // ---- deliver.  LDS executes a wave's operations in order, so the partial sums above are in
    // place before the count below is; the wave that delivers a tile's last unit finishes it.
    unsigned arrived = 0;
    if (lane == 0)
      asm volatile("ds_add_rtn_u32 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)"
                   : "=&v"(arrived) : "v"(ctr_abs + 4 * (1 + slot)), "v"(1u) : "memory");
    arrived = __builtin_amdgcn_readfirstlane(arrived);
    if ((int)arrived == upt - 1) {
      const int tile = (int)blockIdx.x + tl * a.grid;
      const int64_t row = (int64_t)tile * a.rows + j;
      const uint32_t slot_abs = red_abs + (uint32_t)slot * upt * MT * 64;
      // lane (j, kg) adds columns kg, kg + 4, .. of every activation row (four reads per row and matrix
      // in flight at a time); the four groups then meet.  The order is fixed, so the result does not
      // depend on who arrives last.
      float sg[MT], su[MT];
#pragma unroll
      for (int m = 0; m < MT; m++) sg[m] = su[m] = 0.f;
      for (int c = kg; c < nb; c += 16) {
        float r[MT][2][4];
#pragma unroll
        for (int m = 0; m < MT; m++) {
#pragma unroll
          for (int mt = 0; mt < NMAT; mt++) {
            const uint32_t p = slot_abs + (((mt * nb + c) * MT + m) * 16 + j) * 4;
            asm volatile(
                "ds_read_b32 %0, %4\n\t"
                "ds_read_b32 %1, %4 offset:%5\n\t"
                "ds_read_b32 %2, %4 offset:%6\n\t"
                "ds_read_b32 %3, %4 offset:%7"
                : "=&v"(r[m][mt][0]), "=&v"(r[m][mt][1]), "=&v"(r[m][mt][2]), "=&v"(r[m][mt][3])
                : "v"(p), "n"(4 * MT * 64), "n"(8 * MT * 64), "n"(12 * MT * 64)
                : "memory");
          }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int m = 0; m < MT; m++) {
          asm volatile("" : "+v"(r[m][0][0]), "+v"(r[m][0][1]), "+v"(r[m][0][2]), "+v"(r[m][0][3]));
          if (DUAL) asm volatile("" : "+v"(r[m][NMAT - 1][0]), "+v"(r[m][NMAT - 1][1]), "+v"(r[m][NMAT - 1][2]), "+v"(r[m][NMAT - 1][3]));
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const bool ok = c + 4 * i < nb;       // columns past the last read whatever follows: dropped
            sg[m] += ok ? r[m][0][i] : 0.f;
            if (DUAL) su[m] += ok ? r[m][NMAT - 1][i] : 0.f;
          }
        }
      }
      if (norm && !have_rms) {
        // every column has been consumed by now, so every column's sum of squares is in place: lane l
        // takes columns l, l + 64, .. (one LDS read each, all lanes at once), then the lanes meet in a
        // fixed order
#pragma unroll
        for (int m = 0; m < MT; m++) {
          float part = 0.f;
          for (int c = lane; c < nb; c += 64) part += __uint_as_float(lds_read_u32(xq_abs + (uint32_t)(c * MT + m) * kRec + kRecSsq));
          const float tot = dh::wave_sum_uniform(part);
          inv_rms[m] = 1.0f / sqrtf(tot / (float)a.K + a.norm_eps);
        }
      }
#pragma unroll
      for (int m = 0; m < MT; m++) {
        float g = sum_lane_groups(sg[m]), u = 0.f;
        if (DUAL) u = sum_lane_groups(su[m]);
        if (norm) {
          g *= inv_rms[m];
          u *= inv_rms[m];
        }
        if (kg == 0 && j < a.rows && m < a.M && row < a.N) {
          float v;
          if (DUAL) {
            const float act = a.activation == DH_ACT_SILU ? act_silu(g) : act_gelu(g);
            v = act * u * a.alpha;
            if (a.activation == DH_ACT_SILU && a.clamp_max > 0.f) v = fminf(fmaxf(v, -a.clamp_max), a.clamp_max);
          } else {
            v = g * a.alpha;
            if (a.residual) v += a.residual[(int64_t)m * a.N + row];
          }
          if (a.c_f16)
            reinterpret_cast<__half*>(a.C)[(int64_t)m * a.N + row] = __float2half(v);
          else
            reinterpret_cast<float*>(a.C)[(int64_t)m * a.N + row] = v;
        }
      }
      have_rms = true;
      // slot free for the tile nslots further on (after the reads above: same wave, in order)
      if (lane == 0) {
        ctr[1 + slot] = 0u;
        ctr[1 + nslots + slot] = (unsigned)tl / (unsigned)nslots + 1u;
      }
    }
  }
#undef DH_ISSUE
#undef DH_DECODE
}

int env_int(const char* name, int dflt) { return dh::tuning_int(name, dflt); }

template <int MT, bool DUAL, bool VEC, bool AF16 = false>
int launch_i8_vec(I8Args a, const char* op) {
  constexpr int NMAT = DUAL ? 2 : 1;
  size_t cap = kMaxLds;
  auto kern = q4k_gemv_i8_kernel<MT, DUAL, VEC, AF16>;
  static const int env_depth = env_int("DH_GEMV_DEPTH", 0);
  const int ncu = dh::num_cus();
  // rows per tile: the largest count <= 16 that gives every workgroup the same number of tiles
  const int per_cu = (int)dh::ceil_div(a.N, (int64_t)ncu * kTileRows);
  static const int env_rows = env_int("DH_GEMV_ROWS", 0);
  a.rows = std::max(1, std::min(kTileRows, (int)dh::ceil_div(a.N, (int64_t)ncu * per_cu)));
  if (env_rows > 0) a.rows = std::min(kTileRows, env_rows);
  a.nlw = (9 * a.rows + 63) / 64;
  const int64_t ntiles = dh::ceil_div(a.N, a.rows);
  const int grid = (int)std::min<int64_t>(ntiles, ncu);
  a.upt = a.nb * NMAT;
  a.upt_mul = (int)(((1u << 24) + (unsigned)a.upt - 1) / (unsigned)a.upt);
  a.grid = grid;
  a.tiles_base = (int)(ntiles / grid);
  a.tiles_rem = (int)(ntiles % grid);
  const int64_t units = (int64_t)(a.tiles_base + (a.tiles_rem ? 1 : 0)) * a.upt;     // per workgroup, at most
  // the division by multiplication is exact while units * (upt_mul * upt - 2^24) < 2^24, and the
  // kernel forms the product in 32 bits
  if (units * ((int64_t)a.upt_mul * a.upt - (1 << 24)) >= (1 << 24) || units >= (1 << 20) ||
      units * (int64_t)a.upt_mul >= ((int64_t)1 << 32))
    return -1;
  // the kernel forms byte offsets inside a matrix in 32 bits (the last tile's rows are clamped, never read past)
  if (((int64_t)ntiles * a.rows + kTileRows) * a.nb * kBlockBytes >= ((int64_t)1 << 32)) return -1;
  int depth = 1;
  if (env_depth > 0) depth = std::min(kMaxDepth, env_depth);
  // tile slots: the units in flight (16 waves x (depth + 1) draws) span at most this many tiles
  const int need = (kWaves * (kSlotDepth + 1) + a.upt - 1) / a.upt + 2;
  int nslots = 2;
  while (nslots < need) nslots *= 2;
  if (nslots > kMaxSlots) return -1;
  a.nslots = nslots;
  a.slot_shift = 0;
  while ((1 << a.slot_shift) < nslots) a.slot_shift++;
  auto lds_for = [&](int dep) {
    return (size_t)kWaves * dep * kStage + (size_t)a.nb * MT * kRec + kZeroBytes +
           sizeof(float) * nslots * a.upt * MT * 16 + sizeof(unsigned) * (2 + 2 * nslots + a.nb) + kReadAhead * MT;
  };
  while (depth > 1 && lds_for(depth) > cap) depth--;
  if (lds_for(depth) > cap) return -1;
  a.depth = depth;
  {
    const int64_t rec[12] = {a.rows, a.nlw, grid, a.tiles_base, a.tiles_rem, depth, (int64_t)lds_for(depth), a.upt, a.upt_mul,
                             nslots, 0, MT};
    for (int i = 0; i < 12; i++) dh::plan_layout(i, rec[i]);
  }
  if (dh::plan_note(DH_PLAN_GEMV_I8)) return 0;
  static bool attr_set = false;   // once per instantiation: the call costs microseconds
  if (!attr_set) {
    DH_CHECK_HIP(op, hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)cap));
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * kWaves), lds_for(depth), dh::stream(), a);
  DH_CHECK_LAUNCH(op);
  return 0;
}

// Fast path: K a multiple of 4 and 16-byte aligned rows (vector loads of the activations).
template <int MT, bool DUAL>
int launch_i8(const I8Args& a, const char* op) {
  if (a.a_f16) {
    // f16 rows: only the single-matrix product without a norm prologue, K a multiple of 4 and 8-byte
    // aligned rows; anything else is left to the caller (which widens the rows first)
    if constexpr (!DUAL) {
      if ((a.K & 3) == 0 && (reinterpret_cast<uintptr_t>(a.A) & 7) == 0 && !a.norm_weight)
        return launch_i8_vec<MT, false, true, true>(a, op);
    }
    return -1;
  }
  const bool vec = (a.K & 3) == 0 && (reinterpret_cast<uintptr_t>(a.A) & 15) == 0 &&
                   (!a.norm_weight || (reinterpret_cast<uintptr_t>(a.norm_weight) & 15) == 0);
  return vec ? launch_i8_vec<MT, DUAL, true>(a, op) : launch_i8_vec<MT, DUAL, false>(a, op);
}

// Bytes of LDS a launch with MT activation rows needs at ring depth 1 (what launch_i8_vec computes).
size_t i8_lds_bytes(int mt, int nb, int nmat) {
  const int upt = nb * nmat;
  const int need = (kWaves * (kSlotDepth + 1) + upt - 1) / upt + 2;
  int nslots = 2;
  while (nslots < need) nslots *= 2;
  return (size_t)kWaves * kStage + (size_t)nb * mt * kRec + kZeroBytes + sizeof(float) * nslots * upt * mt * 16 +
         sizeof(unsigned) * (2 + 2 * nslots + nb) + kReadAhead * mt;
}

template <bool DUAL>
int launch_mt(int mt, const I8Args& a, const char* op) {
  return mt == 2 ? launch_i8<2, DUAL>(a, op) : launch_i8<1, DUAL>(a, op);
}

// M activation rows in as few passes over the weights as the LDS allows: 2 or 1 rows per pass (the
// rows' operands, 832 bytes per row and super-block column, must fit beside the ring).
template <bool DUAL>
int dispatch_i8(const I8Args& a, const char* op) {
  const size_t c_elem = a.c_f16 ? 2 : 4;
  int mt = 1;
  for (int cand : {2}) {
    if (cand / 2 < a.M && i8_lds_bytes(cand, a.nb, DUAL ? 2 : 1) <= kMaxLds - 4096) mt = cand;
  }
  if (i8_lds_bytes(mt, a.nb, DUAL ? 2 : 1) > kMaxLds - 4096) return -1;
  for (int m0 = 0; m0 < a.M; m0 += mt) {
    I8Args b = a;
    b.M = std::min(mt, a.M - m0);
    b.A = a.a_f16 ? reinterpret_cast<const float*>(reinterpret_cast<const uint16_t*>(a.A) + (int64_t)m0 * a.K)
                  : a.A + (int64_t)m0 * a.K;
    b.C = static_cast<char*>(a.C) + (int64_t)m0 * a.N * c_elem;
    b.residual = a.residual ? a.residual + (int64_t)m0 * a.N : nullptr;
    const int rc = launch_mt<DUAL>(mt, b, op);
    if (rc != 0) return m0 == 0 ? rc : dh::fail(2, "[%s] internal: GEMV pass %d did not launch after pass 0 did", op, m0 / mt);
  }
  return 0;
}

}  // namespace

namespace dh {

int q4k_gemv_i8(const char* op, const float* A, const uint8_t* W, const uint8_t* W2, void* C, int c_f16,
                const float* residual, int M, int N, int K, float alpha, int activation, float clamp_max,
                const float* norm_weight, float norm_eps, int norm_weight_offset, int a_f16) {
  static const int off = env_int("DH_GEMV_I8_OFF", 0);
  // three and more activation rows stay with the f16 matrix-core kernel of q4k_gemv.hip: their
  // operands (832 bytes per row and column) crowd the LDS and the per-row epilogue outweighs the
  // weight stream (measured: 24 against 21 us for the fused gate/up product at M = 4)
  if (off || M < 1 || M > 2) return -1;
  I8Args a{};
  a.A = A; a.W = W; a.W2 = W2; a.C = C; a.residual = residual;
  a.M = M; a.N = N; a.K = K; a.nb = (K + kQK - 1) / kQK;
  a.a_f16 = a_f16;
  a.alpha = alpha; a.c_f16 = c_f16; a.activation = activation; a.clamp_max = clamp_max;
  a.norm_weight = norm_weight; a.norm_eps = norm_eps; a.norm_weight_offset = norm_weight_offset;
  a.status = dh::kernel_status_word();
  return W2 ? dispatch_i8<true>(a, op) : dispatch_i8<false>(a, op);
}

}  // namespace dh
