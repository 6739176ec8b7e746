// Chained Q4_K decode GEMVs: up to four dependent products of ONE activation row in a single launch,
//
//     x_0 given,   x_{p+1} = f_p( W_p . g_p(x_p) )            (p = 0 .. n-1)
//
// with g_p an optional RMSNorm of the input and f_p either  alpha * (.) + residual  or the gated pair
// act(Wg . x) * (Wu . x) * alpha.  This is the dependent run of products between two attentions of a
// decoder layer (o-projection, gate/up, down-projection, the next layer's q/k/v projection), which as
// four launches costs four times the dispatch-to-first-byte floor of a launch with the HBM idle.
//
// One persistent workgroup of 16 waves per compute unit.  Every workgroup owns fixed row tiles of
// every matrix; a work unit is one tile x one 256-weight super-block column (<= 16 rows x 144 bytes).
// Inside a phase the waves draw the workgroup's units from a counter in LDS, one unit in flight per
// wave (global_load_lds into its private ring; a second one in flight was measured slower: the
// stream is bandwidth-bound with sixteen, and a longer first burst only delays the first results).
// A wave that finds no unit left in phase p moves on alone: it requests its first unit of phase p + 1
// (unit `wave`, no draw) BEFORE it waits at the exchange, so while the outputs of phase p travel
// between the workgroups the first sixteen units per compute unit of phase p + 1 are on their way
// into LDS.
//
// Exchange.  The wave that finishes a tile writes its outputs to C and, for every phase but the last,
// publishes them as (value, sequence number) pairs with 8-byte device-scope stores (an 8-byte store
// is single-copy atomic, so a reader that sees the number sees the value).  The consumers, every
// workgroup for the whole vector, read the pairs with device-scope loads and retry until every number
// is the one of this launch and phase.  No counters, no fences, no grid barrier; two buffers in
// turn, so that a phase's outputs are never overwritten before every workgroup has consumed them
// (a workgroup publishes phase p + 1 only after it has consumed phase p, and phase p + 2 can only be
// published after every workgroup has published phase p + 1).  Every wait is bounded: a wave whose
// wait runs into the limit stores a code in the library's status word and leaves, the other waves of
// the workgroup follow, the other workgroups run into their own limits, and the host finds the code at
// its next synchronisation.  The sequence numbers come from a launch counter in device memory that
// the launch itself advances, so a captured graph can replay the launch.
//
// The arithmetic of a unit (int8 matrix cores over activations quantised per 32-element sub-block)
// is that of q4k_gemv_i8.hip; the two share q4k_i8_device.h.
#include <algorithm>
#include <cfloat>
#include <cstdlib>
#include <cstring>

#include "attention_keys.h"
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
constexpr int kStage = 3 * 1024;                   // a wave's ring: one unit (16 rows x 144 bytes = 2304) as three
                                                   // full 64-lane loads of 16 bytes: the third one's lanes past the unit
                                                   // land in the stage's own tail, so no load needs a lane mask
constexpr int kUnitLoads = 3;                     // load instructions of a full unit: ceil(16 rows * 9 pieces / 64 lanes)
constexpr int kMaxPhases = DH_CHAIN_MAX_PHASES;
constexpr int kSlots = 8;                         // tiles whose partial sums may be in LDS at once (a power of two)
constexpr int kSlotShift = 3;
constexpr int kZeroBytes = 144;                   // what a lane without an operand reads
constexpr size_t kMaxLds = 160 * 1024;
constexpr int kMaxChainN = 32768;                 // longest exchanged vector
constexpr int kDefaultSpinLimit = 1 << 17;        // polls of one bounded wait
constexpr int kColsPerPass = 3;                   // columns whose loads a wave has in flight at once in the prologue
// counters in LDS: [p] next unit of phase p to draw, [kCtrArrived + s] units delivered to slot s,
// [kCtrGen + s] tiles completed in slot s, [kCtrAbort] a wave has given up, [kCtrDone + p] tiles of
// phase p this workgroup has finished, then the column flags of the two record areas
constexpr int kCtrNext = 0;
constexpr int kCtrArrived = kMaxPhases;
constexpr int kCtrGen = kCtrArrived + kSlots;
constexpr int kCtrAbort = kCtrGen + kSlots;
constexpr int kCtrDone = kCtrAbort + 1;
constexpr int kCtrFlags = kCtrDone + kMaxPhases;
// a tile's partial sums are read four columns at a time: the last read may reach past the counters
constexpr int kLdsPad = 1024;

#define DH_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
// s_waitcnt with only the vector-memory counter set (6 bits, split 4 + 2 in the encoding).
#define DH_WAIT_VM(k) __builtin_amdgcn_s_waitcnt(((k) & 0xF) | (((k) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

// Waits until at most n (0..3) of this wave's vector-memory operations are outstanding (they
// complete in issue order).
__device__ __forceinline__ void wait_vm_at_most(int n) {
  switch (n) {
    case 1: DH_WAIT_VM(1); break;
    case 2: DH_WAIT_VM(2); break;
    case 3: DH_WAIT_VM(3); break;
    default: DH_WAIT_VM(0); break;
  }
}

struct Phase {
  const uint8_t* W;            // Q4_K rows [N][nb]
  const uint8_t* W2;           // second matrix of a gated pair, or null
  float* C;                    // [N]
  const float* residual;       // [N] or null
  const float* norm_weight;    // [K] or null: RMSNorm of the phase's input
  int N, K, nb, nmat;
  int rows;                    // weight rows per tile (<= 16)
  int nlw;                     // load instructions per unit: ceil(9 * rows / 64)
  int upt;                     // units per tile: nb * nmat
  int upt_mul;                 // ceil(2^24 / upt): u / upt == (u * upt_mul) >> 24 for the unit counts met here
  int tiles_base, tiles_rem;   // tiles per workgroup: floor and remainder of tiles / grid
  int activation, norm_weight_offset;
  int wait_stores;             // a later phase reads this phase's C as its residual
  float alpha, clamp_max, norm_eps;
};

struct ChainArgs {
  Phase ph[kMaxPhases];
  const float* x0;             // [K of phase 0]
  v2u* ll;                     // [2][kMaxChainN] (value, sequence number)
  uint32_t* epoch;             // launch counter (device memory)
  uint32_t* status;            // the library's kernel status word
  int nph;
  int grid;                    // workgroups the tiles are dealt to (the launch may hold fewer: diagnostic)
  int spin_limit;
  int xq_bytes[2];             // bytes of the two record areas (phases 0, 2 / 1, 3)
  int nb_max[2];               // columns of the two areas
  int red_stride;              // floats per tile slot: 16 * the largest units-per-tile
  // phase 0's input as the split-K partial results of a decode attention (null: x0): [H][attn_stride][D + 2]
  // (o..., m, l) per query head and split; the split count is attn_nsplit, or follows the key count
  // on the device as the attention kernels' own does
  const float* attn_ws;
  int attn_H, attn_D, attn_nsplit;
  int attn_stride;             // splits per head in the workspace layout
  dh::DynKeys attn_dyn;
};

__device__ __forceinline__ float wave_max64(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}
__device__ __forceinline__ float wave_sum64(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

__device__ __forceinline__ uint32_t lds_read_u32(uint32_t addr) {
  uint32_t v;
  asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(v) : "v"(addr) : "memory");
  return v;
}

__global__ __launch_bounds__(64 * kWaves, 1) void q4k_gemv_chain_kernel(const ChainArgs a) {
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bid = blockIdx.x;
  // what every phase uses is fetched in one batch here (left alone the compiler fetches an argument
  // where it is first used: a dependent trip to memory each time)
  asm volatile("" :: "s"(a.x0), "s"(a.ll), "s"(a.epoch), "s"(a.status));
  asm volatile("" :: "s"(a.nph), "s"(a.grid), "s"(a.spin_limit), "s"(a.xq_bytes[0]), "s"(a.xq_bytes[1]), "s"(a.nb_max[0]),
               "s"(a.nb_max[1]), "s"(a.red_stride));
  asm volatile("" :: "s"(a.ph[0].norm_weight), "s"(a.ph[0].nb));

  // ---- LDS: ring [16 waves][3072], record areas 0 and 1, zeros [144], partial sums
  // [kSlots][red_stride], counters
  unsigned char* ring = lds;
  unsigned char* xq0 = ring + (size_t)kWaves * kStage;
  unsigned char* xq1 = xq0 + a.xq_bytes[0];
  unsigned char* zeros = xq1 + a.xq_bytes[1];
  float* red = reinterpret_cast<float*>(zeros + kZeroBytes);
  unsigned* ctr = reinterpret_cast<unsigned*>(red + (size_t)kSlots * a.red_stride);
  const int nflags = a.nb_max[0] + a.nb_max[1];
  // (every wave takes unit `wave` of a phase without drawing: the unit counters start behind those)
  for (int i = tid; i < kCtrFlags + nflags; i += 64 * kWaves) ctr[i] = i < kMaxPhases ? (unsigned)kWaves : 0u;
  if (tid >= 64 && tid < 64 + kZeroBytes / 4) reinterpret_cast<uint32_t*>(zeros)[tid - 64] = 0u;

  // the launch counter: requested first, so that it arrives with (ahead of) phase 0's activations and
  // costs no round trip of its own; phase p's outputs carry seq_base + p + 1
  uint32_t epoch_v;
  asm volatile("global_load_dword %0, %1, off" : "=&v"(epoch_v) : "v"(a.epoch) : "memory");
  uint32_t seq_base = 0;
  const int nph = a.nph;

  unsigned char* my_ring = ring + (size_t)wave * kStage;
  const uint32_t ctr_abs = (uint32_t)(uintptr_t)DH_LDS_PTR(ctr);
  const uint32_t abort_addr = ctr_abs + 4 * kCtrAbort;
  const uint32_t red_abs = (uint32_t)(uintptr_t)DH_LDS_PTR(red);
  const uint32_t xq_abs0 = (uint32_t)(uintptr_t)DH_LDS_PTR(xq0), xq_abs1 = (uint32_t)(uintptr_t)DH_LDS_PTR(xq1);

  // A bounded wait ran into its limit: the wave lets its loads land, leaves the code where the host
  // finds it, tells the other waves of the workgroup and ends.
  auto give_up = [&](const uint32_t kind, const int phase) {
    DH_WAIT_VM(0);
    if (lane == 0) {
      __hip_atomic_store(a.status, dh::kstatus_code(kind, (uint32_t)phase, (uint32_t)bid), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_SYSTEM);
      ctr[kCtrAbort] = 1u;
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_endpgm();          // the wave ends here (no barrier follows)
  };

  // ---- a phase's activations: this wave's share is columns (wave - bid) mod 16, + 16, .. (rotated by
  // workgroup so that the workgroups do not all ask for the same lines at the same moment),
  // kColsPerPass of them per pass.  Lane t holds elements 4t .. 4t+3 of a column.  Phase 0 reads x0,
  // written before the launch; later phases read the pairs the other workgroups publish and retry
  // until every sequence number is the expected one.
  struct Cols {
    v4f xr[kColsPerPass], wr[kColsPerPass];
  };
  const int c_first = (wave - bid) & (kWaves - 1);
  auto load_norm = [&](const float* nw, const int nb, const int c0, Cols& R) {
    if (nw == nullptr) return;
#pragma unroll
    for (int i = 0; i < kColsPerPass; i++) {
      const int c = c0 + kWaves * i;
      if (c < nb) {
        const float* q = nw + c * kQK + 4 * lane;
        asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(R.wr[i]) : "v"(q) : "memory");
      }
    }
  };
  auto load_x0 = [&](const int nb, const int c0, Cols& R) {
#pragma unroll
    for (int i = 0; i < kColsPerPass; i++) {
      const int c = c0 + kWaves * i;
      if (c < nb) {
        const float* q = a.x0 + c * kQK + 4 * lane;
        asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(R.xr[i]) : "v"(q) : "memory");
      }
    }
  };
  // Quantises the columns of a pass (their values have landed) and raises their flags.
  auto finish_pass = [&](const int p, const bool norm, const int nwo, const int nb, const int c0, Cols& R) {
    unsigned char* xq = (p & 1) ? xq1 : xq0;
    unsigned* flags = ctr + kCtrFlags + ((p & 1) ? a.nb_max[0] : 0);
#pragma unroll
    for (int i = 0; i < kColsPerPass; i++) {
      const int c = c0 + kWaves * i;
      if (c < nb) {
        asm volatile("" : "+v"(R.xr[i]));
        if (norm) asm volatile("" : "+v"(R.wr[i]));
        float v[4], ss = 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          v[e] = R.xr[i][e];
          if (norm) {
            ss = fmaf(v[e], v[e], ss);
            v[e] *= nwo ? 1.0f + R.wr[i][e] : R.wr[i][e];
          }
        }
        unsigned char* rec = xq + (size_t)c * kRec;
        i8_quantise_store(v, rec, lane);
        if (norm) ss = dh::wave_sum_uniform(ss);
        // LDS executes a wave's operations in order: whoever sees the flag sees the record
        if (lane == 0) {
          reinterpret_cast<float*>(rec)[kRecSsq / 4] = ss;
          flags[c] = (unsigned)p + 1u;
        }
      }
    }
  };

  // the first pass of phase 0: its loads go out before the barrier and before any weights, so that
  // they are at the head of the compute unit's memory queue
  const bool from_attn = a.attn_ws != nullptr;
  Cols first;
  // Phase 0's input from a decode attention's split-K partial results: the first wave of workgroup h
  // merges query head h (out[d] = sum_s e^{m_s - M} o_s[d] / sum_s e^{m_s - M} l_s, the arithmetic and
  // summation order of the attention's own merge kernel) and publishes it as phase "-1" of the
  // exchange; every workgroup then takes phase 0's input from there as it takes a later phase's.
  // Everything the merge reads (of the first 32 splits) is requested here, before the barrier: one
  // trip to memory.  Lane s holds (m, l) of split s, lane t the output dims 2t, 2t + 1.
  constexpr int kMergePre = 32;
  const bool merger = from_attn && wave == 0 && bid < a.attn_H;
  int m_nsplit = 0;
  const float* m_base = nullptr;
  v2f m_ml = {-FLT_MAX, 0.f};
  v2f m_ov[kMergePre];
  if (merger) {
    // the loads do not wait for the split count (with the key count on the device it is one more load):
    // splits past it are read and ignored
    m_base = a.attn_ws + (int64_t)bid * a.attn_stride * (a.attn_D + 2);
    const int smax = a.attn_stride;
    if (lane < smax) {
      const float* q = m_base + (int64_t)lane * (a.attn_D + 2) + a.attn_D;
      asm volatile("global_load_dwordx2 %0, %1, off" : "=&v"(m_ml) : "v"(q) : "memory");
    }
    if (2 * lane < a.attn_D) {
#pragma unroll
      for (int i = 0; i < kMergePre; i++) {
        const float* q = m_base + (int64_t)min(i, smax - 1) * (a.attn_D + 2) + 2 * lane;
        asm volatile("global_load_dwordx2 %0, %1, off" : "=&v"(m_ov[i]) : "v"(q) : "memory");
      }
    }
    m_nsplit = a.attn_nsplit;
    if (a.attn_dyn.kv_len_ptr != nullptr) m_nsplit = dh::dyn_key_range(a.attn_dyn).nsplit;
    m_nsplit = __builtin_amdgcn_readfirstlane(m_nsplit);
  }
  if (!from_attn) {
    load_norm(a.ph[0].norm_weight, a.ph[0].nb, c_first, first);
    load_x0(a.ph[0].nb, c_first, first);
  }

  // counters, flags and the zero area are in place
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

  if (from_attn) {
    DH_WAIT_VM(0);
    asm volatile("" : "+v"(epoch_v));
    seq_base = __builtin_amdgcn_readfirstlane(epoch_v) * 8u;
    if (merger) {
      const int AD = a.attn_D;
      asm volatile("" : "+v"(m_ml));
      const bool has = lane < m_nsplit;
      const float m0 = has ? m_ml[0] : -FLT_MAX, l0 = has ? m_ml[1] : 0.f;
      const float M = wave_max64(m0);
      const float f = has ? __expf(m0 - M) : 0.f;
      const float den = wave_sum64(has ? f * l0 : 0.f);
      const bool dims = 2 * lane < AD;
      float n0 = 0.f, n1 = 0.f;
#pragma unroll
      for (int i = 0; i < kMergePre; i++) {
        asm volatile("" : "+v"(m_ov[i]));
        if (i < m_nsplit) {
          const float fs = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(f), i));
          n0 = fmaf(fs, m_ov[i][0], n0);
          n1 = fmaf(fs, m_ov[i][1], n1);
        }
      }
#pragma unroll 1
      for (int s0 = kMergePre; s0 < m_nsplit; s0 += 16) {
        float2 ov[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int sidx = min(s0 + i, m_nsplit - 1);
          ov[i] = dims ? *reinterpret_cast<const float2*>(m_base + (int64_t)sidx * (AD + 2) + 2 * lane) : make_float2(0.f, 0.f);
        }
#pragma unroll
        for (int i = 0; i < 16; i++) {
          if (s0 + i < m_nsplit) {
            const float fs = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(f), s0 + i));
            n0 = fmaf(fs, ov[i].x, n0);
            n1 = fmaf(fs, ov[i].y, n1);
          }
        }
      }
      if (dims) {
        v2u p0, p1;
        p0.x = __float_as_uint(den > 0.f ? n0 / den : 0.f);
        p1.x = __float_as_uint(den > 0.f ? n1 / den : 0.f);
        p0.y = p1.y = seq_base;
        v2u* dst = a.ll + (size_t)kMaxChainN + (size_t)bid * AD + 2 * lane;
        asm volatile("global_store_dwordx2 %0, %1, off sc1\n\tglobal_store_dwordx2 %0, %2, off offset:8 sc1"
                     :: "v"(dst), "v"(p0), "v"(p1) : "memory");
      }
    }
  }

  // operand addressing (see q4k_gemv_i8.hip): MFMA pair cc covers sub-blocks 4cc .. 4cc+3; lane
  // (i = lane & 15, kg) supplies operand row i = 4g + digit: 16 digit bytes where its row's sub-block is
  // the one its k-slots hold, zeros elsewhere and in the fourth row of every group
  const int j = lane & 15, kg = lane >> 4;
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
  const uint32_t hp = (uint32_t)(uintptr_t)DH_LDS_PTR(my_ring) + (uint32_t)j * kBlockBytes;   // this lane's row header in the ring
  const uint32_t qp = hp + 16 + 32 * (kg >> 1) + 16 * (kg & 1);                               // its 16 nibble bytes of chunk kg >> 1
  const uint32_t sh_lo = 8 * kg;           // bit offset of this lane's byte in the header words

  // What putting a unit's loads in flight needs of its phase.
  struct Stream {
    const uint8_t* W;
    const uint8_t* W2;
    int64_t row_bytes;
    int N, nb, dual, rows, upt, upt_mul;
    // byte offsets inside a weight matrix fit 32 bits (checked on the host): a unit's address is one
    // 64-bit base plus 32-bit scalar arithmetic
    uint32_t wg_off;               // this workgroup's first tile
    uint32_t tile_stride;          // to its next tile
    int rows_left0, rows_round;    // rows from the first tile's first row to the matrix's end; rows per round of tiles
    uint32_t goff[kUnitLoads];     // piece t * 64 + lane of a unit: row q / 9, 16-byte piece q % 9 of that row's super-block
  };
  auto stream_of = [&](const Phase& Q) {
    Stream S;
    S.W = Q.W; S.W2 = Q.W2; S.N = Q.N; S.nb = Q.nb; S.dual = Q.nmat - 1; S.rows = Q.rows; S.upt = Q.upt; S.upt_mul = Q.upt_mul;
    S.row_bytes = (int64_t)Q.nb * kBlockBytes;
    S.wg_off = (uint32_t)bid * (uint32_t)Q.rows * (uint32_t)S.row_bytes;
    S.tile_stride = (uint32_t)a.grid * (uint32_t)Q.rows * (uint32_t)S.row_bytes;
    S.rows_left0 = Q.N - bid * Q.rows;
    S.rows_round = a.grid * Q.rows;
#pragma unroll
    for (int t = 0; t < kUnitLoads; t++) {
      const int q = t * 64 + lane, r = q / 9;
      // (lanes past the tile's pieces fetch piece 0 again: their 16 bytes land behind the unit, unread)
      S.goff[t] = q < 9 * S.rows ? (uint32_t)(r * S.row_bytes + (q - r * 9) * 16) : 0u;
    }
    return S;
  };
  // Unit u of a workgroup's phase = (tile ordinal tl, matrix, column): u = (tl * nmat + mat) * nb + col.
#define DH_DECODE(S_, u_, tl_, mat_, col_)                                   \
  const int tl_ = (int)(((unsigned)(u_) * (unsigned)(S_).upt_mul) >> 24);    \
  const int r__##tl_ = (u_) - tl_ * (S_).upt;                                \
  const int mat_ = ((S_).dual && r__##tl_ >= (S_).nb) ? 1 : 0;               \
  const int col_ = r__##tl_ - mat_ * (S_).nb;
  // Puts the loads of unit u in flight into the wave's ring.
  auto issue = [&](const Stream& S, const int u) {
    DH_DECODE(S, u, itl, imat, icol)
    const uint32_t off = S.wg_off + (uint32_t)itl * S.tile_stride + (uint32_t)icol * kBlockBytes;
    const uint8_t* base = (imat ? S.W2 : S.W) + off;
    const int rows_left = S.rows_left0 - itl * S.rows_round;
    if (rows_left >= S.rows) {
#pragma unroll
      for (int t = 0; t < kUnitLoads; t++) {
        // (the offset is made opaque here so that its widening to 64 bits is not hoisted out of the unit
        // loop: only then does the load take the form scalar base + 32-bit lane offset, with no vector add)
        uint32_t g = S.goff[t];
        asm volatile("" : "+v"(g));
        __builtin_amdgcn_global_load_lds(base + g, DH_LDS_PTR(my_ring + t * 1024), 16, 0, 0);
      }
    } else {
#pragma unroll
      for (int t = 0; t < kUnitLoads; t++) {
        const int q = t * 64 + lane, rr = q / 9;
        const int64_t o = (int64_t)min(rr, rows_left - 1) * S.row_bytes + (q - rr * 9) * 16;
        __builtin_amdgcn_global_load_lds(base + o, DH_LDS_PTR(my_ring + t * 1024), 16, 0, 0);
      }
    }
  };

  // ---- phase 0's activations come from x0: the wave's first unit (unit `wave`, no draw) is requested
  // behind their loads, and only they are waited for
  int cur = 0x7fffffff;                     // the unit in the ring (>= its phase's total: none)
  if (!from_attn) {
    const Phase& Q = a.ph[0];
    const Stream S = stream_of(Q);
    const int total = (Q.tiles_base + (bid < Q.tiles_rem ? 1 : 0)) * Q.upt;
    const int nb = Q.nb, nwo = Q.norm_weight_offset;
    const float* const nw = Q.norm_weight;
    cur = wave < total ? wave : 0x7fffffff;
    if (cur < total) issue(S, cur);
    wait_vm_at_most(cur < total ? Q.nlw : 0);
    asm volatile("" : "+v"(epoch_v));
    seq_base = __builtin_amdgcn_readfirstlane(epoch_v) * 8u;
    finish_pass(0, nw != nullptr, nwo, nb, c_first, first);
#pragma unroll 1
    for (int c0 = c_first + kWaves * kColsPerPass; c0 < nb; c0 += kWaves * kColsPerPass) {
      Cols R;
      load_norm(nw, nb, c0, R);
      load_x0(nb, c0, R);
      DH_WAIT_VM(0);
      finish_pass(0, nw != nullptr, nwo, nb, c0, R);
    }
  }

  // ---- phase by phase.  A wave enters phase p when phase p - 1 has no unit left for it to draw.
  // On the way in it requests its first unit of the phase (the weights do not depend on the
  // exchange, and its ring is free), then prepares its share of the phase's activations, which the
  // other waves count on whether or not this wave gets a unit of the phase.
  int tb = 0;                               // tile ordinal (over all phases) of the phase's first tile in this workgroup
  int prev_ntl = 0;                         // tiles of this workgroup in the previous phase
#pragma unroll 1
  for (int p = 0; p < nph; p++) {
    const Phase& Q = a.ph[p];
    const Stream S = stream_of(Q);
    // what the unit loop itself reads is fetched together; what only a tile's end needs is fetched there
    asm volatile("" :: "s"(S.W), "s"(S.W2), "s"(S.N), "s"(S.nb), "s"(S.dual), "s"(S.rows), "s"(S.upt), "s"(S.upt_mul));
    asm volatile("" :: "s"(S.wg_off), "s"(S.tile_stride), "s"(S.rows_left0), "s"(S.rows_round));
    const int nb = S.nb, upt = S.upt;
    const float* const nw = Q.norm_weight;
    const bool norm = nw != nullptr;
    const int ntl = Q.tiles_base + (bid < Q.tiles_rem ? 1 : 0);
    const int total = ntl * upt;                       // units of this workgroup in this phase
    const uint32_t xq_abs = (p & 1) ? xq_abs1 : xq_abs0;
    const uint32_t flags_abs = ctr_abs + 4 * (kCtrFlags + ((p & 1) ? a.nb_max[0] : 0));
    const uint32_t next_abs = ctr_abs + 4 * (kCtrNext + p);
    const uint32_t flag_want = (uint32_t)p + 1u;
    const bool last_phase = p == nph - 1;

    if (p > 0 || from_attn) {
      // ---- the wave's first unit of the phase: unit `wave`, no draw
      cur = wave < total ? wave : 0x7fffffff;
      if (cur < total) issue(S, cur);

      // ---- the phase's activations
      const int nwo = Q.norm_weight_offset;
      const v2u* src = a.ll + (size_t)((p - 1) & 1) * kMaxChainN;
      const uint32_t want = seq_base + (uint32_t)p;
      // Not before this workgroup has finished its own tiles of the previous phase: the workgroups run
      // the same work at the same pace, so until then the others have not finished theirs either, and
      // polls that cannot succeed yet would only compete with the weight stream for the memory system.
      if (p > 0) {
        const uint32_t done_addr = ctr_abs + 4 * (kCtrDone + p - 1);
        int spins = 0;
        while (__builtin_amdgcn_readfirstlane(lds_read_u32(done_addr)) < (unsigned)prev_ntl) {
          if (++spins > a.spin_limit * 8 || __builtin_amdgcn_readfirstlane(lds_read_u32(abort_addr)) != 0u)
            give_up(DH_KSTATUS_SLOT_WAIT, p);
          __builtin_amdgcn_s_sleep(4);
        }
      }
#pragma unroll 1
      for (int c0 = c_first; c0 < nb; c0 += kWaves * kColsPerPass) {
        Cols R;
        v4u la[kColsPerPass], lb[kColsPerPass];
        load_norm(nw, nb, c0, R);
        int spins = 0;
        for (;;) {
#pragma unroll
          for (int i = 0; i < kColsPerPass; i++) {
            const int c = c0 + kWaves * i;
            if (c < nb) {
              const v2u* q = src + c * kQK + 4 * lane;
              asm volatile("global_load_dwordx4 %0, %2, off sc1\n\tglobal_load_dwordx4 %1, %2, off offset:16 sc1"
                           : "=&v"(la[i]), "=&v"(lb[i]) : "v"(q) : "memory");
            }
          }
          DH_WAIT_VM(0);
          bool ok = true;
#pragma unroll
          for (int i = 0; i < kColsPerPass; i++) {
            const int c = c0 + kWaves * i;
            if (c < nb) {
              asm volatile("" : "+v"(la[i]), "+v"(lb[i]));
              ok = ok && la[i].y == want && la[i].w == want && lb[i].y == want && lb[i].w == want;
            }
          }
          if (__builtin_amdgcn_ballot_w64(!ok) == 0ull) break;
          if (++spins > a.spin_limit || __builtin_amdgcn_readfirstlane(lds_read_u32(abort_addr)) != 0u) {
            give_up(DH_KSTATUS_EXCHANGE_WAIT, p);
          }
          __builtin_amdgcn_s_sleep(8);
        }
#pragma unroll
        for (int i = 0; i < kColsPerPass; i++)
          R.xr[i] = v4f{__uint_as_float(la[i].x), __uint_as_float(la[i].z), __uint_as_float(lb[i].x), __uint_as_float(lb[i].z)};
        finish_pass(p, norm, nwo, nb, c0, R);
      }
    }

    // ---- the phase's units
    float inv_rms = 1.f;
    bool have_rms = false;
#pragma unroll 1
    for (;;) {
      if (cur >= total) break;              // draws only grow: nothing behind this one either
      DH_DECODE(S, cur, tl, mat, col)
      const int tord = tb + tl;                         // tile ordinal of the workgroup, over all phases
      const int slot = tord & (kSlots - 1);
      // draw the unit that will go into the ring once this one has been read (the answer is collected
      // with the reads below)
      unsigned nxt = 0;
      if (lane == 0) asm volatile("ds_add_rtn_u32 %0, %1, %2" : "=&v"(nxt) : "v"(next_abs), "v"(1u) : "memory");
      DH_WAIT_VM(0);
      const uint32_t rec = xq_abs + (uint32_t)col * kRec;
      const uint32_t gen_addr = ctr_abs + 4 * (kCtrGen + slot);
      const uint32_t flag_addr = flags_abs + 4 * col;
      v4u h, q0, q1;
      v4i ax[2][2];
      v2f sx, xinv;
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
      // the column's operands, read at once on the expectation that its flag is up; re-read below if it was not
#define DH_READ_OPERANDS()                                                                        \
      do {                                                                                        \
        const uint32_t pa = rec * a_mul[0] + a_off[0], pb = rec * a_mul[1] + a_off[1], ps = rec + kRecSums + 4 * kg; \
        asm volatile(                                                                             \
            "ds_read_b128 %0, %6\n\t"                                                             \
            "ds_read_b128 %1, %7\n\t"                                                             \
            "ds_read_b128 %2, %6 offset:128\n\t"                                                  \
            "ds_read_b128 %3, %7 offset:128\n\t"                                                  \
            "ds_read2_b32 %4, %8 offset1:4\n\t"                                                   \
            "ds_read2_b32 %5, %8 offset0:8 offset1:12"                                            \
            : "=&v"(ax[0][0]), "=&v"(ax[0][1]), "=&v"(ax[1][0]), "=&v"(ax[1][1]), "=&v"(sx), "=&v"(xinv) \
            : "v"(pa), "v"(pb), "v"(ps)                                                           \
            : "memory");                                                                          \
      } while (0)
#define DH_TIE_OPERANDS() asm volatile("" : "+v"(ax[0][0]), "+v"(ax[0][1]), "+v"(ax[1][0]), "+v"(ax[1][1]), "+v"(sx), "+v"(xinv))
      DH_READ_OPERANDS();
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(h), "+v"(q0), "+v"(q1), "+v"(gen), "+v"(flag), "+v"(nxt) :: "memory");
      DH_TIE_OPERANDS();
      if (__builtin_amdgcn_readfirstlane(flag) != flag_want) {
        int spins = 0;
        do {
          __builtin_amdgcn_s_sleep(2);
          flag = lds_read_u32(flag_addr);
          if (++spins > a.spin_limit * 8 || __builtin_amdgcn_readfirstlane(lds_read_u32(abort_addr)) != 0u) break;
        } while (__builtin_amdgcn_readfirstlane(flag) != flag_want);
        if (__builtin_amdgcn_readfirstlane(flag) != flag_want) give_up(DH_KSTATUS_COLUMN_WAIT, p);
        DH_READ_OPERANDS();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        DH_TIE_OPERANDS();
      }
#undef DH_READ_OPERANDS
#undef DH_TIE_OPERANDS
      // the ring is free again: put the loads of the unit drawn above in flight
      cur = (int)__builtin_amdgcn_readfirstlane(nxt);
      if (cur < total) issue(S, cur);

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
      // wait (never, in practice) until the tile that used this slot kSlots tiles ago is written out
      {
        const unsigned want = (unsigned)tord >> kSlotShift;
        int spins = 0;
        while (__builtin_amdgcn_readfirstlane(gen) != want) {
          __builtin_amdgcn_s_sleep(1);
          gen = lds_read_u32(gen_addr);
          if (++spins > a.spin_limit * 8 || __builtin_amdgcn_readfirstlane(lds_read_u32(abort_addr)) != 0u) break;
        }
        if (__builtin_amdgcn_readfirstlane(gen) != want) give_up(DH_KSTATUS_SLOT_WAIT, p);
      }
      v4i dd[2];
#pragma unroll
      for (int cc = 0; cc < 2; cc++) {
        v4i t = __builtin_amdgcn_mfma_i32_16x16x64_i8(ax[cc][0], blo[cc], v4i{0, 0, 0, 0}, 0, 0, 0);
        dd[cc] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ax[cc][1], bhi[cc], t, 0, 0, 0);
      }
      // the four lane groups hold different sub-blocks of the same 16 rows
      const float sres = sum_lane_groups(i8_unit_term(dd[0], dd[1], sc_a, sc_b, mn_a, mn_b, d, dmin, sx, xinv));
      if (lane < 16) red[(size_t)slot * a.red_stride + (mat * nb + col) * 16 + lane] = sres;

      // ---- deliver.  LDS executes a wave's operations in order, so the partial sums above are in
      // place before the count below is; the wave that delivers a tile's last unit finishes it.
      unsigned arrived = 0;
      if (lane == 0)
        asm volatile("ds_add_rtn_u32 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(arrived) : "v"(ctr_abs + 4 * (kCtrArrived + slot)), "v"(1u) : "memory");
      arrived = __builtin_amdgcn_readfirstlane(arrived);
      if ((int)arrived == upt - 1) {
        const int tile = bid + tl * a.grid;
        const int rows = S.rows, N = S.N, dual = S.dual;
        const int64_t row = (int64_t)tile * rows + j;
        const uint32_t slot_abs = red_abs + (uint32_t)slot * a.red_stride * 4;
        // lane (j, kg) adds columns kg, kg + 4, .. (four reads in flight at a time); the four groups then
        // meet.  The order is fixed, so the result does not depend on who arrives last.
        float sg = 0.f, su = 0.f;
        for (int c = kg; c < nb; c += 16) {
          float r[2][4];
#pragma unroll
          for (int mt = 0; mt < 2; mt++) {
            if (mt == 0 || S.dual) {
              const uint32_t q = slot_abs + ((mt * nb + c) * 16 + j) * 4;
              asm volatile(
                  "ds_read_b32 %0, %4\n\t"
                  "ds_read_b32 %1, %4 offset:256\n\t"
                  "ds_read_b32 %2, %4 offset:512\n\t"
                  "ds_read_b32 %3, %4 offset:768"
                  : "=&v"(r[mt][0]), "=&v"(r[mt][1]), "=&v"(r[mt][2]), "=&v"(r[mt][3])
                  : "v"(q)
                  : "memory");
            } else {
              r[mt][0] = r[mt][1] = r[mt][2] = r[mt][3] = 0.f;
            }
          }
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0][0]), "+v"(r[0][1]), "+v"(r[0][2]), "+v"(r[0][3]) :: "memory");
          asm volatile("" : "+v"(r[1][0]), "+v"(r[1][1]), "+v"(r[1][2]), "+v"(r[1][3]));
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const bool ok = c + 4 * i < nb;       // columns past the last read whatever follows: dropped
            sg += ok ? r[0][i] : 0.f;
            su += ok ? r[1][i] : 0.f;
          }
        }
        sg = sum_lane_groups(sg);
        su = sum_lane_groups(su);
        if (norm) {
          if (!have_rms) {
            // every column has been consumed by now, so every column's sum of squares is in place: lane l
            // takes columns l, l + 64, .. (one LDS read each, all lanes at once), then the lanes meet in a
            // fixed order (the single-product kernel's)
            float part = 0.f;
            for (int c = lane; c < nb; c += 64) part += __uint_as_float(lds_read_u32(xq_abs + (uint32_t)c * kRec + kRecSsq));
            const float tot = dh::wave_sum_uniform(part);
            inv_rms = 1.0f / sqrtf(tot / (float)Q.K + Q.norm_eps);
            have_rms = true;
          }
          sg *= inv_rms;
          su *= inv_rms;
        }
        if (kg == 0 && j < rows && row < N) {
          float v;
          if (dual) {
            const int activation = Q.activation;
            const float clamp_max = Q.clamp_max;
            const float act = activation == DH_ACT_SILU ? act_silu(sg) : act_gelu(sg);
            v = act * su * Q.alpha;
            if (activation == DH_ACT_SILU && clamp_max > 0.f) v = fminf(fmaxf(v, -clamp_max), clamp_max);
          } else {
            v = sg * Q.alpha;
            const float* const residual = Q.residual;
            // device-scope load: an earlier phase of this launch may have written the residual
            if (residual) v += __hip_atomic_load(const_cast<float*>(residual) + row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
          __hip_atomic_store(Q.C + row, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (!last_phase) {
            v2u pr;
            pr.x = __float_as_uint(v);
            pr.y = seq_base + (uint32_t)p + 1u;
            v2u* dst = a.ll + (size_t)(p & 1) * kMaxChainN + row;
            asm volatile("global_store_dwordx2 %0, %1, off sc1" :: "v"(dst), "v"(pr) : "memory");
          }
        }
        // a later phase reads these outputs as its residual: they are in memory before this wave goes on
        if (Q.wait_stores) DH_WAIT_VM(0);
        // slot free for the tile kSlots further on (after the reads above: same wave, in order)
        if (lane == 0) {
          ctr[kCtrArrived + slot] = 0u;
          ctr[kCtrGen + slot] = ((unsigned)tord >> kSlotShift) + 1u;
          unsigned was;
          asm volatile("ds_add_rtn_u32 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)" : "=&v"(was) : "v"(ctr_abs + 4 * (kCtrDone + p)), "v"(1u) : "memory");
        }
        // the launch counter moves on once: the workgroup that owns the last phase's first tile does it
        if (last_phase && bid == 0 && tl == 0 && lane == 0) *a.epoch = (seq_base >> 3) + 1u;
      }
    }
    prev_ntl = ntl;
    tb += ntl;
  }
#undef DH_DECODE
}

// ---- host side ----------------------------------------------------------------------------------
v2u* g_ll = nullptr;          // exchange pairs, 2 x kMaxChainN
uint32_t* g_epoch = nullptr;  // launch counter
bool g_coresident = false;

struct Plan {
  ChainArgs a;
  size_t lds;
};

int make_plan(const char* op, const float* d_x0, const dh_chain_attn_source* src, const dh_chain_phase* ph, int n, Plan* out) {
  if (n < 1 || n > kMaxPhases) return dh::fail(1, "[%s] a chain holds 1..%d products, got %d", op, kMaxPhases, n);
  if ((!d_x0 && !src) || !ph) return dh::fail(1, "[%s] null pointer", op);
  if (reinterpret_cast<uintptr_t>(d_x0) & 15) return dh::fail(1, "[%s] x0 must be 16-byte aligned", op);
  ChainArgs& a = out->a;
  memset(&a, 0, sizeof(a));
  const int ncu = dh::num_cus();
  a.grid = ncu;
  a.nph = n;
  a.x0 = d_x0;
  a.ll = g_ll;
  a.epoch = g_epoch;
  a.status = dh::kernel_status_word();
  a.spin_limit = kDefaultSpinLimit;
  int max_upt = 0, min_upt = 1 << 30;
  for (int p = 0; p < n; p++) {
    const dh_chain_phase& s = ph[p];
    Phase& P = a.ph[p];
    if (s.N <= 0 || s.K <= 0) return dh::fail(1, "[%s] product %d: dimensions must be positive: N=%d, K=%d", op, p, s.N, s.K);
    if (s.K % kQK) return dh::fail(1, "[%s] product %d: K=%d must be a multiple of 256 in a chain", op, p, s.K);
    if (p > 0 && s.K != ph[p - 1].N)
      return dh::fail(1, "[%s] product %d takes K=%d inputs but product %d makes N=%d outputs", op, p, s.K, p - 1, ph[p - 1].N);
    if (s.N > kMaxChainN || s.K > kMaxChainN) return dh::fail(1, "[%s] product %d: N and K are limited to %d in a chain", op, p, kMaxChainN);
    if (!s.d_W || !s.d_C) return dh::fail(1, "[%s] product %d: null pointer", op, p);
    if ((reinterpret_cast<uintptr_t>(s.d_W) | reinterpret_cast<uintptr_t>(s.d_W2)) & 15)
      return dh::fail(1, "[%s] product %d: weight pointers must be 16-byte aligned", op, p);
    if (s.d_norm_weight && (reinterpret_cast<uintptr_t>(s.d_norm_weight) & 15))
      return dh::fail(1, "[%s] product %d: the norm weights must be 16-byte aligned", op, p);
    if (s.d_W2 && s.activation != DH_ACT_SILU && s.activation != DH_ACT_GELU)
      return dh::fail(1, "[%s] product %d: unknown activation %d", op, p, s.activation);
    if (s.d_W2 && s.d_residual) return dh::fail(1, "[%s] product %d: a gated pair takes no residual", op, p);
    P.W = static_cast<const uint8_t*>(s.d_W);
    P.W2 = static_cast<const uint8_t*>(s.d_W2);
    P.C = s.d_C;
    P.residual = s.d_residual;
    P.norm_weight = s.d_norm_weight;
    P.N = s.N; P.K = s.K; P.nb = s.K / kQK; P.nmat = s.d_W2 ? 2 : 1;
    P.activation = s.activation; P.norm_weight_offset = s.norm_weight_offset;
    P.alpha = s.alpha; P.clamp_max = s.swiglu_limit; P.norm_eps = s.norm_eps;
    // rows per tile: the largest count <= 16 that gives every workgroup the same number of tiles
    const int per_cu = (int)dh::ceil_div(s.N, (int64_t)ncu * kTileRows);
    P.rows = std::max(1, std::min(kTileRows, (int)dh::ceil_div(s.N, (int64_t)ncu * per_cu)));
    P.nlw = (9 * P.rows + 63) / 64;
    const int64_t ntiles = dh::ceil_div(s.N, P.rows);
    P.upt = P.nb * P.nmat;
    P.upt_mul = (int)(((1u << 24) + (unsigned)P.upt - 1) / (unsigned)P.upt);
    P.tiles_base = (int)(ntiles / ncu);
    P.tiles_rem = (int)(ntiles % ncu);
    const int64_t units = (int64_t)(P.tiles_base + (P.tiles_rem ? 1 : 0)) * P.upt;
    // the division by multiplication is exact while units * (upt_mul * upt - 2^24) < 2^24
    if (units * ((int64_t)P.upt_mul * P.upt - (1 << 24)) >= (1 << 24) || units >= (1 << 20) ||
        units * (int64_t)P.upt_mul >= ((int64_t)1 << 32))
      return dh::fail(1, "[%s] product %d: N=%d, K=%d is too large for a chain", op, p, s.N, s.K);
    max_upt = std::max(max_upt, P.upt);
    min_upt = std::min(min_upt, P.upt);
    a.nb_max[p & 1] = std::max(a.nb_max[p & 1], P.nb);
    // outputs that a later product reads back as its residual must have reached memory by then
    for (int q = p + 1; q < n; q++)
      if (ph[q].d_residual == s.d_C) P.wait_stores = 1;
    // a product may not overwrite what an earlier or later one of the launch still reads elsewhere
    if (d_x0 && s.d_C == d_x0) return dh::fail(1, "[%s] product %d writes over the chain's input", op, p);
  }
  // the units in flight (16 waves x 2 draws) must not span more tiles than there are slots
  if ((kWaves * 2 + min_upt - 1) / min_upt + 2 > kSlots)
    return dh::fail(1, "[%s] K=%d is too short for a chain (at least 1536)", op, min_upt * kQK);
  if (src) {
    // the first product's input is the merge of a decode attention's split-K partial results
    const int ncus = dh::num_cus();
    if (!src->d_workspace) return dh::fail(1, "[%s] the attention workspace is null", op);
    if (reinterpret_cast<uintptr_t>(src->d_workspace) & 7) return dh::fail(1, "[%s] the attention workspace must be 8-byte aligned", op);
    if (src->H <= 0 || src->Hkv <= 0 || src->H % src->Hkv) return dh::fail(1, "[%s] attention heads %d/%d", op, src->H, src->Hkv);
    if (src->D != 64 && src->D != 128) return dh::fail(1, "[%s] headDim %d not supported (64, 128)", op, src->D);
    if (src->H * src->D != ph[0].K)
      return dh::fail(1, "[%s] the attention makes %d x %d values but product 0 takes K=%d", op, src->H, src->D, ph[0].K);
    if (src->H > ncus) return dh::fail(1, "[%s] %d query heads need as many workgroups (%d)", op, src->H, ncus);
    const int one_per_cu = dh::attn_one_per_cu(ncus, src->Hkv);
    int max_splits;
    if (src->d_kv_len) {
      if (reinterpret_cast<uintptr_t>(src->d_kv_len) & 3) return dh::fail(1, "[%s] the key-count pointer must be 4-byte aligned", op);
      if (src->max_kv_len < 1 || src->sliding_window < 0 || src->kv_start < 0)
        return dh::fail(1, "[%s] need max_kv_len >= 1, slidingWindow >= 0, kvStart >= 0", op);
      max_splits = dh::max_splits_upto(one_per_cu, src->max_kv_len);
      // the arithmetic of dh_attn_decode_qkv_kvlen_partials: causal, the query at the last key
      a.attn_dyn = dh::DynKeys{src->d_kv_len, src->max_kv_len, 1, -1, src->sliding_window, src->kv_start, 1, one_per_cu};
    } else {
      if (src->nsplit < 1) return dh::fail(1, "[%s] nsplit must be at least 1", op);
      max_splits = src->nsplit;
    }
    if (max_splits > 64) return dh::fail(1, "[%s] up to 64 splits are merged in the chain (this call may have %d)", op, max_splits);
    a.attn_ws = static_cast<const float*>(src->d_workspace);
    a.attn_H = src->H;
    a.attn_D = src->D;
    a.attn_nsplit = src->nsplit;
    a.attn_stride = max_splits;
  }
  a.xq_bytes[0] = a.nb_max[0] * kRec;
  a.xq_bytes[1] = a.nb_max[1] * kRec;
  a.red_stride = 16 * max_upt;
  out->lds = (size_t)kWaves * kStage + a.xq_bytes[0] + a.xq_bytes[1] + kZeroBytes +
             sizeof(float) * kSlots * a.red_stride + sizeof(unsigned) * (kCtrFlags + a.nb_max[0] + a.nb_max[1]) + kLdsPad;
  if (out->lds > kMaxLds)
    return dh::fail(1, "[%s] the chain's activations do not fit the LDS (%zu of %zu bytes)", op, out->lds, kMaxLds);
  return 0;
}

int launch(const char* op, Plan& plan, int workgroups) {
  auto kern = q4k_gemv_chain_kernel;
  static bool attr_set = false;
  if (!attr_set) {
    DH_CHECK_HIP(op, hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)kMaxLds));
    // the workgroups wait for each other: every one of them must be resident at once
    int per_cu = 0;
    DH_CHECK_HIP(op, hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kern), 64 * kWaves,
                                                                  kMaxLds));
    g_coresident = per_cu >= 1;
    attr_set = true;
  }
  if (!g_coresident) return dh::fail(1, "[%s] the device cannot hold one workgroup of the chain per compute unit", op);
  hipLaunchKernelGGL(kern, dim3(workgroups), dim3(64 * kWaves), plan.lds, dh::stream(), plan.a);
  DH_CHECK_LAUNCH(op);
  return 0;
}

}  // namespace

namespace dh {

int gemv_chain_init(int) {
  DH_CHECK_HIP("dh_init", hipMalloc(reinterpret_cast<void**>(&g_ll), (size_t)2 * kMaxChainN * sizeof(v2u)));
  DH_CHECK_HIP("dh_init", hipMalloc(reinterpret_cast<void**>(&g_epoch), 256));
  DH_CHECK_HIP("dh_init", hipMemset(g_ll, 0, (size_t)2 * kMaxChainN * sizeof(v2u)));
  const uint32_t one = 1u;
  DH_CHECK_HIP("dh_init", hipMemcpy(g_epoch, &one, 4, hipMemcpyHostToDevice));
  return 0;
}

void gemv_chain_release() {
  if (g_ll) (void)hipFree(g_ll);
  if (g_epoch) (void)hipFree(g_epoch);
  g_ll = nullptr;
  g_epoch = nullptr;
}

// After a launch that gave up: sequence numbers of the abandoned launch may be anywhere in the
// exchange area and the counter has not moved on; start over (the stream is idle when this runs).
void gemv_chain_reset() {
  if (!g_ll) return;
  (void)hipMemset(g_ll, 0, (size_t)2 * kMaxChainN * sizeof(v2u));
  uint32_t e = 0;
  if (hipMemcpy(&e, g_epoch, 4, hipMemcpyDeviceToHost) != hipSuccess) e = 0;
  e += 2u;
  (void)hipMemcpy(g_epoch, &e, 4, hipMemcpyHostToDevice);
}

}  // namespace dh

extern "C" {

int dh_q4k_gemv_chain(const float* d_x0, const dh_chain_phase* phases, int n_phases) {
  const char* op = "dh_q4k_gemv_chain";
  DH_REQUIRE_INIT(op);
  Plan plan;
  if (!d_x0) return dh::fail(1, "[%s] null pointer", op);
  if (int rc = make_plan(op, d_x0, nullptr, phases, n_phases, &plan)) return rc;
  return launch(op, plan, plan.a.grid);
}

int dh_q4k_gemv_chain_attn_supported(int H, int Hkv, int D, int max_kv_len) {
  if (!dh::ready() || H <= 0 || Hkv <= 0 || H % Hkv || (D != 64 && D != 128) || max_kv_len < 1) return 0;
  const int ncus = dh::num_cus();
  return H <= ncus && dh::max_splits_upto(dh::attn_one_per_cu(ncus, Hkv), max_kv_len) <= 64 ? 1 : 0;
}

int dh_q4k_gemv_chain_attn(const dh_chain_attn_source* source, const dh_chain_phase* phases, int n_phases) {
  const char* op = "dh_q4k_gemv_chain_attn";
  DH_REQUIRE_INIT(op);
  if (!source) return dh::fail(1, "[%s] null pointer", op);
  Plan plan;
  if (int rc = make_plan(op, nullptr, source, phases, n_phases, &plan)) return rc;
  return launch(op, plan, plan.a.grid);
}

int dh_q4k_gemv_chain_limited(const float* d_x0, const dh_chain_phase* phases, int n_phases, int workgroups,
                              int spin_limit) {
  const char* op = "dh_q4k_gemv_chain_limited";
  DH_REQUIRE_INIT(op);
  Plan plan;
  if (!d_x0) return dh::fail(1, "[%s] null pointer", op);
  if (int rc = make_plan(op, d_x0, nullptr, phases, n_phases, &plan)) return rc;
  if (workgroups < 1 || workgroups > plan.a.grid)
    return dh::fail(1, "[%s] workgroups must be 1..%d", op, plan.a.grid);
  if (spin_limit < 1 || spin_limit > kDefaultSpinLimit) return dh::fail(1, "[%s] spin_limit must be 1..%d", op, kDefaultSpinLimit);
  plan.a.spin_limit = spin_limit;
  return launch(op, plan, workgroups);
}

}  // extern "C"
