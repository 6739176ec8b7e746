// Shared host-side plumbing of libdopplerhip: error reporting, the single stream every op
// enqueues on, and launch helpers.  gfx950 only.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <type_traits>

#include "../../include/doppler_hip.h"

namespace dh {

constexpr int kQK = 256;           // weights per Q4_K super-block
constexpr int kBlockBytes = 144;   // bytes per super-block
constexpr int kWave = 64;

// Records a message for dh_last_error() and returns the code to hand back to the caller.
int fail(int code, const char* fmt, ...);
hipStream_t stream();
bool ready();
int num_cus();
// Scratch for the split-K prefill GEMM's partial products (allocated by dh_init, shared by all
// launches on the library's stream, which run in order).
float* splitk_workspace(size_t* bytes);
// Per-row scale factors of the prefill GEMM's activations: capacity rows x (multiplier, inverse).
float* gemm_row_scale();
// Packed f16 activations of the prefill GEMM (rows x K rounded up to 64 halves).
void* gemm_packed_a(size_t* bytes);
int gemm_row_scale_capacity();
// f32 copy of f16 activations handed to dh_q4k_matmul (allocated by dh_init; one matmul at a time
// uses it, in stream order).
float* widened_activations(size_t* bytes);

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Tile shapes, ring depths and kernel families have ONE setting in the library as it is built.  A
// build with -DDH_TUNING_ENV (measurements only, never the shipped library) reads overrides of the
// same names from the environment.
inline const char* tuning_env(const char* name) {
#ifdef DH_TUNING_ENV
  return getenv(name);
#else
  (void)name;
  return nullptr;
#endif
}
inline int tuning_int(const char* name, int dflt) {
  const char* e = tuning_env(name);
  return e ? atoi(e) : dflt;
}
inline double tuning_double(const char* name, double dflt) {
  const char* e = tuning_env(name);
  return e ? atof(e) : dflt;
}

// ---- planning (dh_q4k_matmul_plan) ------------------------------------------------------------
// While a plan is being made on this thread the dispatchers run as usual on the shape alone: ready()
// holds, num_cus() is the planned device's count, and every launch site reports its kernel family
// through plan_note() instead of launching (true = planning, return without touching the device).
bool plan_note(int family);
// What the noted launch would have been: entry i of the plan's layout record (see dh_q4k_gemv_layout).
void plan_layout(int i, int64_t value);
void plan_begin(int num_cus);
int plan_end();
const int64_t* plan_layout_record();

// ---- kernel status word ---------------------------------------------------------------------
// Kernels that wait on other waves or workgroups bound every such wait; a wave whose wait runs
// into its limit stores a code here and leaves.  The word lives in pinned host memory that the
// device can write, so the host can look at it for free after every stream synchronisation
// (dh_sync, dh_download, dh_upload, dh_free), which then fail with the decoded message.
#define DH_KSTATUS_COLUMN_WAIT 1u     // GEMV: a column's activation operands never arrived
#define DH_KSTATUS_SLOT_WAIT 2u       // GEMV: a tile slot was never released
#define DH_KSTATUS_EXCHANGE_WAIT 3u   // chained GEMV: another workgroup's outputs never arrived
uint32_t* kernel_status_word();
// Reads and clears the word (call only after the stream has been synchronised); non-zero -> fail().
int check_kernel_status(const char* op);
// chained GEMV (q4k_gemv_chain.hip): called when a launch has reported a failed wait, so that the
// next launch starts from a clean exchange area.
void gemv_chain_reset();
// chained GEMV: exchange area and launch counter (allocated by dh_init, freed with the runtime).
int gemv_chain_init(int device);
void gemv_chain_release();

// Matrix-core GEMM for prefill-sized batches (q4k_gemm.hip).  `serves`: M >= 16, K a multiple
// of 4, A 16-byte aligned.
bool q4k_gemm_serves(int M, int K, const void* A);
// norm_weight != null: every row of A goes through RMSNorm (weights norm_weight, or 1 + them) on its
// way into the packed operand.
int q4k_gemm(const char* op, const float* A, const uint8_t* W, void* C, int c_f16, int M, int N, int K,
             float alpha, const float* residual, const float* norm_weight = nullptr, float norm_eps = 0.f,
             int norm_weight_offset = 0);
int q4k_gemm_gate_up(const char* op, const float* A, const uint8_t* Wg, const uint8_t* Wu, float* C, int M,
                     int hidden, int inter, int activation, float alpha, float clamp_max,
                     const float* norm_weight = nullptr, float norm_eps = 0.f, int norm_weight_offset = 0);

// ---- captured decode steps (dh_graph_*, dh_runtime.hip) ---------------------------------------
// One decode attention call made while a graph was being captured: everything needed to redo its
// host-side arithmetic (visible key range, key splits, rotary table row, appended cache row) for
// another position and patch the two kernel nodes it became.
struct GraphAttnCall {
  int qkv;                 // 1: dh_attn_decode_qkv, 0: dh_attn_decode
  const float* q;          // Q [H][D], or the stacked qkv projection
  const float* qw;
  const float* kw;
  const float* cos;
  const float* sin;
  void* K;
  void* V;
  float* O;
  int H, Hkv, D;
  int kv_len, start_pos;   // at capture time
  int causal;
  int rotary_dim, interleaved, weight_offset, use_norm;
  float eps, scale, softcap;
  int sliding_window, kv_start, kv_layout;
  void* ws;
  size_t ws_capacity;      // bytes behind ws when the library knows them (its own scratch), else 0
  hipGraphNode_t split_node, merge_node;
};
// A dh_check_finiteness call recorded during a capture: its step number follows the position.
struct GraphFiniteCall {
  const void* input;
  int dtype;
  int64_t size;
  uint32_t* status;
  uint32_t layer, step;    // step at capture time
  float abs_threshold;
  unsigned grid;
  hipGraphNode_t node;
};
struct Graph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  int position = 0;                       // position the node parameters currently stand at
  int captured_position = 0;
  int max_position = -1;                  // largest position the step's buffers cover, when the caller declared it
  GraphAttnCall* attn = nullptr;
  int n_attn = 0, cap_attn = 0;
  GraphFiniteCall* fin = nullptr;
  int n_fin = 0, cap_fin = 0;
};
// The graph being captured on the op stream, or null.
Graph* capturing_graph();
// attention.hip: records a call for the graph being captured (no-op outside a capture).
void graph_note_attention(const GraphAttnCall& call);
// attention.hip: finds the kernel nodes of the recorded calls in the captured graph / patches them for `position`.
int attn_graph_bind(Graph* g);
int attn_graph_set_position(Graph* g, int position);
// elementwise.hip: the same for the finiteness checks of a captured step (their step number is a
// launch argument: a replay at position p reports captured step + p - captured position).
void graph_note_finiteness(const GraphFiniteCall& call);
int finite_graph_bind(Graph* g);
int finite_graph_set_position(Graph* g, int position);

// Looks up, once per device, the address of the fixed device array that dh_attn_decode_static uses
// for its split partials (attention.hip).  Called by dh_init with the device current.
int attn_static_scratch_init(int device);

// Decode GEMV on the int8 matrix cores (q4k_gemv_i8.hip): C = alpha * A . W^T + residual, or with W2
// the gated pair act(A . W^T) * (A . W2^T) * alpha; norm_weight != null normalises A's rows first.
// Returns -1 when the shape is not served (the caller then takes another kernel), 0 on success.
// a_f16: A holds f16 rows (single matrix, no norm prologue, K a multiple of 4, rows 8-byte aligned;
// -1 otherwise), widened exactly as they are loaded.
int q4k_gemv_i8(const char* op, const float* A, const uint8_t* W, const uint8_t* W2, void* C, int c_f16,
                const float* residual, int M, int N, int K, float alpha, int activation, float clamp_max,
                const float* norm_weight, float norm_eps, int norm_weight_offset, int a_f16 = 0);
// The same product for up to 8 activation rows in one pass over the weights, on the f16 matrix cores
// (q4k_gemv_rows.hip).  Same arguments and return values.
int q4k_gemv_rows(const char* op, const float* A, const uint8_t* W, const uint8_t* W2, void* C, int c_f16,
                  const float* residual, int M, int N, int K, float alpha, int activation, float clamp_max,
                  const float* norm_weight, float norm_eps, int norm_weight_offset, int a_f16 = 0);

}  // namespace dh

namespace dh {
// kind in the top 4 bits (never zero), phase of a chained launch below it, workgroup in the low 24.
__host__ __device__ inline uint32_t kstatus_code(uint32_t kind, uint32_t phase, uint32_t block) {
  return (kind << 28) | ((phase & 0xFu) << 24) | (block & 0xFFFFFFu);
}
}  // namespace dh

#ifdef __HIPCC__
namespace dh {
// Sum over the 64 lanes of a wave, returned wave-uniform: DPP row shifts inside each 16-lane
// row (no LDS traffic), then the four row totals travel through scalar registers.
__device__ __forceinline__ float wave_sum_uniform(float v) {
  auto shr = [](float x, auto ctrl) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), decltype(ctrl)::value, 0xF, 0xF, false));
  };
  v += shr(v, std::integral_constant<int, 0x111>{});
  v += shr(v, std::integral_constant<int, 0x112>{});
  v += shr(v, std::integral_constant<int, 0x114>{});
  v += shr(v, std::integral_constant<int, 0x118>{});
  const int b = __float_as_int(v);
  return (__int_as_float(__builtin_amdgcn_readlane(b, 15)) + __int_as_float(__builtin_amdgcn_readlane(b, 31))) +
         (__int_as_float(__builtin_amdgcn_readlane(b, 47)) + __int_as_float(__builtin_amdgcn_readlane(b, 63)));
}
}  // namespace dh
#endif

#define DH_REQUIRE_INIT(op)                                                     \
  do {                                                                          \
    if (!dh::ready()) return dh::fail(1, "[%s] dh_init has not been called", op); \
  } while (0)

#define DH_CHECK_HIP(op, expr)                                                       \
  do {                                                                               \
    hipError_t e_ = (expr);                                                          \
    if (e_ != hipSuccess)                                                            \
      return dh::fail(2, "[%s] %s failed: %s", op, #expr, hipGetErrorString(e_));    \
  } while (0)

// After a kernel launch: surfaces launch-configuration errors at the call site.
#define DH_CHECK_LAUNCH(op) DH_CHECK_HIP(op, hipGetLastError())
