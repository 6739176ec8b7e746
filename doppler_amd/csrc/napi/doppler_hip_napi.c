/*
 * Node-API binding of libdopplerhip.so for the JavaScript host code.
 *
 * Thin by design: one JS function per C-ABI entry point, device pointers travel as BigInt,
 * a non-zero return code becomes a thrown Error carrying dh_last_error() -- the reference's
 * ops report failures as `throw new Error('[Op] ...')` and nothing else.  Built with plain
 * gcc against /usr/include/node/node_api.h (N-API version <= 8, Node 12 compatible).
 */
#include <node_api.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "doppler_hip.h"

#define MAX_ARGS 24

static napi_value fail(napi_env env, const char* msg) {
  napi_throw_error(env, NULL, msg);
  return NULL;
}

static int get_args(napi_env env, napi_callback_info info, size_t want, napi_value* argv) {
  size_t argc = MAX_ARGS;
  if (napi_get_cb_info(env, info, &argc, argv, NULL, NULL) != napi_ok) return 0;
  if (argc < want) {
    napi_throw_type_error(env, NULL, "doppler_hip: too few arguments");
    return 0;
  }
  return 1;
}

/* BigInt -> device pointer; null/undefined -> NULL. */
static int arg_ptr(napi_env env, napi_value v, void** out) {
  napi_valuetype t;
  napi_typeof(env, v, &t);
  if (t == napi_null || t == napi_undefined) { *out = NULL; return 1; }
  if (t != napi_bigint) { napi_throw_type_error(env, NULL, "doppler_hip: device pointer must be a BigInt or null"); return 0; }
  uint64_t u = 0; bool lossless = false;
  napi_get_value_bigint_uint64(env, v, &u, &lossless);
  *out = (void*)(uintptr_t)u;
  return 1;
}
static int arg_i64(napi_env env, napi_value v, int64_t* out) {
  double d;
  if (napi_get_value_double(env, v, &d) != napi_ok) { napi_throw_type_error(env, NULL, "doppler_hip: number expected"); return 0; }
  *out = (int64_t)d;
  return 1;
}
static int arg_int(napi_env env, napi_value v, int* out) {
  int64_t t;
  if (!arg_i64(env, v, &t)) return 0;
  *out = (int)t;
  return 1;
}
static int arg_f32(napi_env env, napi_value v, float* out) {
  double d;
  if (napi_get_value_double(env, v, &d) != napi_ok) { napi_throw_type_error(env, NULL, "doppler_hip: number expected"); return 0; }
  *out = (float)d;
  return 1;
}

static napi_value ret_rc(napi_env env, int rc) {
  if (rc != 0) return fail(env, dh_last_error());
  napi_value u;
  napi_get_undefined(env, &u);
  return u;
}
static napi_value ret_ptr(napi_env env, void* p) {
  napi_value v;
  napi_create_bigint_uint64(env, (uint64_t)(uintptr_t)p, &v);
  return v;
}
static napi_value ret_num(napi_env env, double d) {
  napi_value v;
  napi_create_double(env, d, &v);
  return v;
}

#define FN(name) static napi_value name(napi_env env, napi_callback_info info)
#define ARGS(n) napi_value a[MAX_ARGS]; if (!get_args(env, info, n, a)) return NULL
#define P(i, var) void* var; if (!arg_ptr(env, a[i], &var)) return NULL
#define I(i, var) int var; if (!arg_int(env, a[i], &var)) return NULL
#define L(i, var) int64_t var; if (!arg_i64(env, a[i], &var)) return NULL
#define F(i, var) float var; if (!arg_f32(env, a[i], &var)) return NULL

/* ---- captured decode steps ---- */
FN(js_graph_begin) { (void)info; return ret_rc(env, dh_graph_begin()); }
FN(js_graph_end) {
  ARGS(1); I(0, position);
  void* g = NULL;
  if (dh_graph_end(position, &g) != 0) return fail(env, dh_last_error());
  return ret_ptr(env, g);
}
FN(js_graph_launch) { ARGS(2); P(0, g); I(1, position); return ret_rc(env, dh_graph_launch(g, position)); }
FN(js_graph_set_max_position) { ARGS(2); P(0, g); I(1, position); return ret_rc(env, dh_graph_set_max_position(g, position)); }
FN(js_graph_prepare) { ARGS(2); P(0, g); I(1, position); return ret_rc(env, dh_graph_prepare(g, position)); }
FN(js_graph_destroy) { ARGS(1); P(0, g); return ret_rc(env, dh_graph_destroy(g)); }

/* ---- device / memory ---- */
FN(js_init) { ARGS(1); I(0, dev); return ret_rc(env, dh_init(dev)); }
FN(js_shutdown) { (void)info; return ret_rc(env, dh_shutdown()); }
FN(js_sync) { (void)info; return ret_rc(env, dh_sync()); }
FN(js_malloc) {
  ARGS(1); L(0, bytes);
  void* p = NULL;
  if (dh_malloc((size_t)bytes, &p) != 0) return fail(env, dh_last_error());
  return ret_ptr(env, p);
}
FN(js_free) { ARGS(1); P(0, p); return ret_rc(env, dh_free(p)); }
/* upload(dst, dstOffset, ArrayBuffer|TypedArray|Buffer) */
static int arg_bytes(napi_env env, napi_value v, void** data, size_t* len) {
  bool is = false;
  napi_is_typedarray(env, v, &is);
  if (is) {
    napi_typedarray_type tt; size_t n; napi_value ab; size_t off;
    napi_get_typedarray_info(env, v, &tt, &n, data, &ab, &off);
    static const size_t esz[] = {1, 1, 1, 2, 2, 4, 4, 4, 8, 8, 8};
    *len = n * esz[tt];
    return 1;
  }
  napi_is_arraybuffer(env, v, &is);
  if (is) { napi_get_arraybuffer_info(env, v, data, len); return 1; }
  napi_is_buffer(env, v, &is);
  if (is) { napi_get_buffer_info(env, v, data, len); return 1; }
  napi_is_dataview(env, v, &is);
  if (is) { napi_value ab; size_t off; napi_get_dataview_info(env, v, len, data, &ab, &off); return 1; }
  napi_throw_type_error(env, NULL, "doppler_hip: ArrayBuffer or typed array expected");
  return 0;
}
FN(js_upload) {
  ARGS(3); P(0, dst); L(1, off);
  void* data; size_t len;
  if (!arg_bytes(env, a[2], &data, &len)) return NULL;
  return ret_rc(env, dh_upload(dst, (size_t)off, data, len));
}
/* download(src, srcOffset, bytes) -> ArrayBuffer (waits for queued work) */
FN(js_download) {
  ARGS(3); P(0, src); L(1, off); L(2, bytes);
  void* data = NULL; napi_value ab;
  if (napi_create_arraybuffer(env, (size_t)bytes, &data, &ab) != napi_ok) return fail(env, "doppler_hip: ArrayBuffer allocation failed");
  if (dh_download(data, src, (size_t)off, (size_t)bytes) != 0) return fail(env, dh_last_error());
  return ab;
}
FN(js_copy) { ARGS(5); P(0, d); L(1, doff); P(2, s); L(3, soff); L(4, n); return ret_rc(env, dh_copy(d, (size_t)doff, s, (size_t)soff, (size_t)n)); }
FN(js_fill_zero) { ARGS(3); P(0, d); L(1, off); L(2, n); return ret_rc(env, dh_fill_zero(d, (size_t)off, (size_t)n)); }
FN(js_event_create) { (void)info; void* e = NULL; if (dh_event_create(&e) != 0) return fail(env, dh_last_error()); return ret_ptr(env, e); }
FN(js_event_record) { ARGS(1); P(0, e); return ret_rc(env, dh_event_record(e)); }
FN(js_event_elapsed_ms) {
  ARGS(2); P(0, s); P(1, e);
  float ms = 0;
  if (dh_event_elapsed_ms(s, e, &ms) != 0) return fail(env, dh_last_error());
  return ret_num(env, ms);
}
FN(js_event_destroy) { ARGS(1); P(0, e); return ret_rc(env, dh_event_destroy(e)); }
FN(js_event_synchronize) { ARGS(1); P(0, e); return ret_rc(env, dh_event_synchronize(e)); }
/* hostAlloc(bytes) -> {ptr: BigInt, view: ArrayBuffer over the pinned memory (valid until hostFree(ptr))} */
FN(js_host_alloc) {
  ARGS(1); L(0, bytes);
  void* p = NULL;
  if (dh_host_alloc((size_t)bytes, &p) != 0) return fail(env, dh_last_error());
  napi_value obj, view;
  if (napi_create_external_arraybuffer(env, p, (size_t)bytes, NULL, NULL, &view) != napi_ok || napi_create_object(env, &obj) != napi_ok) {
    dh_host_free(p);
    return fail(env, "doppler_hip: could not wrap the pinned memory");
  }
  napi_set_named_property(env, obj, "ptr", ret_ptr(env, p));
  napi_set_named_property(env, obj, "view", view);
  return obj;
}
FN(js_host_free) { ARGS(1); P(0, p); return ret_rc(env, dh_host_free(p)); }
/* downloadAsync(hostPtr, hostOffset, src, srcOffset, bytes): enqueued behind the ops so far, returns at once */
FN(js_download_async) {
  ARGS(5); P(0, h); L(1, hoff); P(2, src); L(3, off); L(4, bytes);
  return ret_rc(env, dh_download_async((char*)h + hoff, src, (size_t)off, (size_t)bytes));
}

/* ---- ops (argument order = the C ABI's) ---- */
FN(js_q4k_dequant) { ARGS(3); P(0, w); L(1, nb); P(2, o); return ret_rc(env, dh_q4k_dequant(w, nb, (float*)o)); }
FN(js_q4k_matmul) {
  ARGS(10); P(0, A); I(1, adt); P(2, W); P(3, C); I(4, cdt); I(5, M); I(6, N); I(7, K); F(8, alpha); P(9, res);
  return ret_rc(env, dh_q4k_matmul(A, adt, W, C, cdt, M, N, K, alpha, res));
}
FN(js_q4k_matmul_rmsnorm) {
  ARGS(12); P(0, A); P(1, nw); F(2, eps); I(3, off); P(4, W); P(5, C); I(6, cdt); I(7, M); I(8, N); I(9, K);
  F(10, alpha); P(11, res);
  return ret_rc(env, dh_q4k_matmul_rmsnorm((const float*)A, (const float*)nw, eps, off, W, C, cdt, M, N, K, alpha, res));
}
FN(js_q4k_ffn_gate_up_rmsnorm) {
  ARGS(13); P(0, x); P(1, nw); F(2, eps); I(3, off); P(4, wg); P(5, wu); P(6, o); I(7, M); I(8, hid); I(9, inter);
  I(10, act); F(11, alpha); F(12, lim);
  return ret_rc(env, dh_q4k_ffn_gate_up_rmsnorm((const float*)x, (const float*)nw, eps, off, wg, wu, (float*)o, M, hid,
                                                inter, act, alpha, lim));
}
FN(js_q4k_ffn_gate_up) {
  ARGS(10); P(0, x); P(1, wg); P(2, wu); P(3, o); I(4, M); I(5, hid); I(6, inter); I(7, act); F(8, alpha); F(9, lim);
  return ret_rc(env, dh_q4k_ffn_gate_up((const float*)x, wg, wu, (float*)o, M, hid, inter, act, alpha, lim));
}
FN(js_f16w_matmul) {
  ARGS(7); P(0, A); P(1, W); P(2, C); I(3, M); I(4, N); I(5, K); F(6, alpha);
  return ret_rc(env, dh_f16w_matmul((const float*)A, W, (float*)C, M, N, K, alpha));
}
FN(js_lmhead_argmax_workspace_bytes) { ARGS(1); I(0, v); return ret_num(env, (double)dh_lmhead_argmax_workspace_bytes(v)); }
FN(js_lmhead_argmax_f16) {
  ARGS(10); P(0, h); P(1, E); I(2, vocab); I(3, hid); L(4, pad); F(5, cap); P(6, ws); P(7, tok); I(8, idx); P(9, logits);
  return ret_rc(env, dh_lmhead_argmax_f16((const float*)h, E, vocab, hid, pad, cap, ws, (uint32_t*)tok, idx, (float*)logits));
}
FN(js_lmhead_argmax_f16_rmsnorm) {
  ARGS(13); P(0, h); P(1, nw); F(2, eps); I(3, off); P(4, E); I(5, vocab); I(6, hid); L(7, pad); F(8, cap); P(9, ws);
  P(10, tok); I(11, idx); P(12, logits);
  return ret_rc(env, dh_lmhead_argmax_f16_rmsnorm((const float*)h, (const float*)nw, eps, off, E, vocab, hid, pad, cap, ws,
                                                  (uint32_t*)tok, idx, (float*)logits));
}
FN(js_attn_decode_workspace_bytes) { ARGS(3); I(0, H); I(1, D); I(2, kv); return ret_num(env, (double)dh_attn_decode_workspace_bytes(H, D, kv)); }
FN(js_attn_decode) {
  ARGS(16); P(0, Q); P(1, K); P(2, V); P(3, O); I(4, H); I(5, Hkv); I(6, D); I(7, kvLen); F(8, scale); I(9, causal);
  I(10, startPos); F(11, cap); I(12, win); I(13, kvStart); I(14, layout); P(15, ws);
  return ret_rc(env, dh_attn_decode((const float*)Q, K, V, (float*)O, H, Hkv, D, kvLen, scale, causal, startPos, cap, win,
                                    kvStart, layout, ws));
}
FN(js_attn_decode_static) {
  ARGS(15); P(0, Q); P(1, K); P(2, V); P(3, O); I(4, H); I(5, Hkv); I(6, D); I(7, kvLen); F(8, scale); I(9, causal);
  I(10, startPos); F(11, cap); I(12, win); I(13, kvStart); I(14, layout);
  return ret_rc(env, dh_attn_decode_static((const float*)Q, K, V, (float*)O, H, Hkv, D, kvLen, scale, causal, startPos, cap,
                                           win, kvStart, layout));
}
FN(js_attn_decode_static_max_bytes) { (void)info; return ret_num(env, (double)dh_attn_decode_static_max_bytes()); }
FN(js_attn_decode_qkv_supported) {
  ARGS(5); I(0, H); I(1, Hkv); I(2, D); I(3, rd); I(4, inter);
  return ret_num(env, (double)dh_attn_decode_qkv_supported(H, Hkv, D, rd, inter));
}
FN(js_attn_decode_qkv) {
  ARGS(23); P(0, qkv); P(1, qw); P(2, kw); P(3, c); P(4, s); P(5, ck); P(6, cv); P(7, O); I(8, H); I(9, Hkv); I(10, D);
  I(11, start); I(12, rd); I(13, inter); F(14, eps); I(15, woff); I(16, useNorm); F(17, scale); F(18, cap); I(19, win);
  I(20, kvStart); I(21, layout); P(22, ws);
  return ret_rc(env, dh_attn_decode_qkv((const float*)qkv, (const float*)qw, (const float*)kw, (const float*)c,
                                        (const float*)s, ck, cv, (float*)O, H, Hkv, D, start, rd, inter, eps, woff,
                                        useNorm, scale, cap, win, kvStart, layout, ws));
}
FN(js_attn_decode_kvlen) {
  ARGS(17); P(0, Q); P(1, K); P(2, V); P(3, O); I(4, H); I(5, Hkv); I(6, D); P(7, kvLenPtr); I(8, maxKvLen); F(9, scale);
  I(10, causal); I(11, startPos); F(12, cap); I(13, win); I(14, kvStart); I(15, layout); P(16, ws);
  return ret_rc(env, dh_attn_decode_kvlen((const float*)Q, K, V, (float*)O, H, Hkv, D, (const uint32_t*)kvLenPtr, maxKvLen,
                                          scale, causal, startPos, cap, win, kvStart, layout, ws));
}
FN(js_attn_decode_qkv_kvlen) {
  ARGS(24); P(0, qkv); P(1, qw); P(2, kw); P(3, c); P(4, s); P(5, ck); P(6, cv); P(7, O); I(8, H); I(9, Hkv); I(10, D);
  P(11, kvLenPtr); I(12, maxKvLen); I(13, rd); I(14, inter); F(15, eps); I(16, woff); I(17, useNorm); F(18, scale);
  F(19, cap); I(20, win); I(21, kvStart); I(22, layout); P(23, ws);
  return ret_rc(env, dh_attn_decode_qkv_kvlen((const float*)qkv, (const float*)qw, (const float*)kw, (const float*)c,
                                              (const float*)s, ck, cv, (float*)O, H, Hkv, D, (const uint32_t*)kvLenPtr,
                                              maxKvLen, rd, inter, eps, woff, useNorm, scale, cap, win, kvStart, layout, ws));
}
/* the splits left unmerged: returns the split count */
FN(js_attn_decode_qkv_partials) {
  ARGS(22); P(0, qkv); P(1, qw); P(2, kw); P(3, c); P(4, s); P(5, ck); P(6, cv); I(7, H); I(8, Hkv); I(9, D);
  I(10, startPos); I(11, rd); I(12, inter); F(13, eps); I(14, woff); I(15, useNorm); F(16, scale); F(17, cap);
  I(18, win); I(19, kvStart); I(20, layout); P(21, ws);
  int nsplit = 0;
  if (dh_attn_decode_qkv_partials((const float*)qkv, (const float*)qw, (const float*)kw, (const float*)c, (const float*)s, ck,
                                  cv, H, Hkv, D, startPos, rd, inter, eps, woff, useNorm, scale, cap, win, kvStart, layout,
                                  ws, &nsplit) != 0)
    return fail(env, dh_last_error());
  return ret_num(env, nsplit);
}
FN(js_attn_decode_qkv_kvlen_partials) {
  ARGS(23); P(0, qkv); P(1, qw); P(2, kw); P(3, c); P(4, s); P(5, ck); P(6, cv); I(7, H); I(8, Hkv); I(9, D);
  P(10, kvLenPtr); I(11, maxKvLen); I(12, rd); I(13, inter); F(14, eps); I(15, woff); I(16, useNorm); F(17, scale);
  F(18, cap); I(19, win); I(20, kvStart); I(21, layout); P(22, ws);
  return ret_rc(env, dh_attn_decode_qkv_kvlen_partials((const float*)qkv, (const float*)qw, (const float*)kw, (const float*)c,
                                                       (const float*)s, ck, cv, H, Hkv, D, (const uint32_t*)kvLenPtr,
                                                       maxKvLen, rd, inter, eps, woff, useNorm, scale, cap, win, kvStart,
                                                       layout, ws));
}
/* ---- chained GEMVs: the structs travel as bytes laid out by the caller (sizes checked here) ---- */
FN(js_chain_struct_sizes) {
  (void)info;
  napi_value arr, v;
  napi_create_array_with_length(env, 2, &arr);
  napi_create_uint32(env, (uint32_t)sizeof(dh_chain_phase), &v); napi_set_element(env, arr, 0, v);
  napi_create_uint32(env, (uint32_t)sizeof(dh_chain_attn_source), &v); napi_set_element(env, arr, 1, v);
  return arr;
}
FN(js_q4k_gemv_chain) {
  ARGS(3); P(0, x0); I(2, n);
  void* ph = NULL; size_t len = 0;
  if (!arg_bytes(env, a[1], &ph, &len)) return NULL;
  if (n < 0 || len < (size_t)n * sizeof(dh_chain_phase)) return fail(env, "[q4kGemvChain] the phase bytes are shorter than n_phases structs");
  return ret_rc(env, dh_q4k_gemv_chain((const float*)x0, (const dh_chain_phase*)ph, n));
}
FN(js_q4k_gemv_chain_attn) {
  ARGS(3); I(2, n);
  void* src = NULL; void* ph = NULL; size_t slen = 0, len = 0;
  if (!arg_bytes(env, a[0], &src, &slen) || !arg_bytes(env, a[1], &ph, &len)) return NULL;
  if (slen < sizeof(dh_chain_attn_source)) return fail(env, "[q4kGemvChainAttn] the source bytes are shorter than the struct");
  if (n < 0 || len < (size_t)n * sizeof(dh_chain_phase)) return fail(env, "[q4kGemvChainAttn] the phase bytes are shorter than n_phases structs");
  return ret_rc(env, dh_q4k_gemv_chain_attn((const dh_chain_attn_source*)src, (const dh_chain_phase*)ph, n));
}
FN(js_q4k_gemv_chain_attn_supported) {
  ARGS(4); I(0, H); I(1, Hkv); I(2, D); I(3, maxKvLen);
  return ret_num(env, dh_q4k_gemv_chain_attn_supported(H, Hkv, D, maxKvLen));
}
FN(js_attn_prefill) {
  ARGS(14); P(0, Q); P(1, K); P(2, V); P(3, O); I(4, T); I(5, H); I(6, Hkv); I(7, D); I(8, kvLen); F(9, scale);
  I(10, causal); I(11, startPos); F(12, cap); I(13, win);
  return ret_rc(env, dh_attn_prefill((const float*)Q, K, V, (float*)O, T, H, Hkv, D, kvLen, scale, causal, startPos, cap, win));
}
FN(js_rmsnorm) {
  ARGS(12); P(0, x); P(1, w); I(2, wdt); P(3, o); I(4, batch); I(5, hid); F(6, eps); I(7, woff); P(8, pre); P(9, post);
  P(10, prenorm); F(11, oscale);
  return ret_rc(env, dh_rmsnorm((const float*)x, w, wdt, (float*)o, batch, hid, eps, woff, (const float*)pre,
                                (const float*)post, (float*)prenorm, oscale));
}
FN(js_rmsnorm_qk) {
  ARGS(13); P(0, q); P(1, k); P(2, qw); I(3, qwdt); P(4, kw); I(5, kwdt); P(6, qo); P(7, ko); I(8, qrows); I(9, krows);
  I(10, hd); F(11, eps); I(12, woff);
  return ret_rc(env, dh_rmsnorm_qk((const float*)q, (const float*)k, qw, qwdt, kw, kwdt, (float*)qo, (float*)ko, qrows,
                                   krows, hd, eps, woff));
}
FN(js_rmsnorm_sandwich_pair) {
  ARGS(12); P(0, x); P(1, r); P(2, pw); I(3, pwdt); P(4, qw); I(5, qwdt); P(6, po); P(7, qo); I(8, batch); I(9, hid);
  F(10, eps); I(11, woff);
  return ret_rc(env, dh_rmsnorm_sandwich_pair((const float*)x, (const float*)r, pw, pwdt, qw, qwdt, (float*)po, (float*)qo,
                                              batch, hid, eps, woff));
}
FN(js_residual_rmsnorm_pair) {
  ARGS(11); P(0, x); P(1, r); P(2, w); I(3, wdt); P(4, ro); P(5, no); I(6, batch); I(7, hid); F(8, eps); I(9, woff);
  F(10, scale);
  return ret_rc(env, dh_residual_rmsnorm_pair((const float*)x, (const float*)r, w, wdt, (float*)ro, (float*)no, batch, hid,
                                              eps, woff, scale));
}
FN(js_rope) {
  ARGS(10); P(0, x); P(1, c); P(2, s); I(3, seq); I(4, heads); I(5, hd); I(6, rd); I(7, span); I(8, inter); I(9, start);
  return ret_rc(env, dh_rope((float*)x, (const float*)c, (const float*)s, seq, heads, hd, rd, span, inter, start));
}
FN(js_rope_qk) {
  ARGS(12); P(0, q); P(1, k); P(2, c); P(3, s); I(4, seq); I(5, qh); I(6, kvh); I(7, hd); I(8, rd); I(9, span); I(10, inter);
  I(11, start);
  return ret_rc(env, dh_rope_qk((float*)q, (float*)k, (const float*)c, (const float*)s, seq, qh, kvh, hd, rd, span, inter,
                                start));
}
FN(js_qkv_norm_rope_kvwrite) {
  ARGS(19); P(0, qkv); P(1, qw); P(2, kw); P(3, c); P(4, s); P(5, qo); P(6, ck); P(7, cv); I(8, T); I(9, H); I(10, Hkv);
  I(11, D); I(12, start); I(13, rd); I(14, inter); F(15, eps); I(16, woff); L(17, dst); I(18, useNorm);
  return ret_rc(env, dh_qkv_norm_rope_kvwrite((const float*)qkv, (const float*)qw, (const float*)kw, (const float*)c,
                                              (const float*)s, (float*)qo, ck, cv, T, H, Hkv, D, start, rd, inter, eps,
                                              woff, dst, useNorm));
}
FN(js_kv_write_f16) {
  ARGS(7); P(0, k); P(1, v); P(2, ck); P(3, cv); L(4, so); L(5, dof); L(6, n);
  return ret_rc(env, dh_kv_write_f16((const float*)k, (const float*)v, ck, cv, so, dof, n));
}
FN(js_residual_add) { ARGS(5); P(0, x); P(1, y); P(2, o); L(3, n); F(4, s); return ret_rc(env, dh_residual_add((const float*)x, (const float*)y, (float*)o, n, s)); }
FN(js_split_qkv) {
  ARGS(8); P(0, x); P(1, q); P(2, k); P(3, v); I(4, t); I(5, qs); I(6, ks); I(7, vs);
  return ret_rc(env, dh_split_qkv((const float*)x, (float*)q, (float*)k, (float*)v, t, qs, ks, vs));
}
FN(js_bias_add) {
  ARGS(7); P(0, d); P(1, b); I(2, bdt); L(3, t); I(4, dim); L(5, doff); L(6, boff);
  return ret_rc(env, dh_bias_add((float*)d, b, bdt, t, dim, doff, boff));
}
FN(js_scale) { ARGS(4); P(0, x); P(1, o); L(2, n); F(3, s); return ret_rc(env, dh_scale((const float*)x, (float*)o, n, s)); }
FN(js_gather_f16) {
  ARGS(7); P(0, ids); P(1, tab); P(2, o); I(3, T); I(4, hid); I(5, vocab); I(6, ioff);
  return ret_rc(env, dh_gather_f16((const uint32_t*)ids, tab, (float*)o, T, hid, vocab, ioff));
}
FN(js_act_gate) { ARGS(6); P(0, g); P(1, u); P(2, o); L(3, n); I(4, act); F(5, lim); return ret_rc(env, dh_act_gate((const float*)g, (const float*)u, (float*)o, n, act, lim)); }
FN(js_act_gate_rowsplit) { ARGS(6); P(0, in); P(1, o); I(2, T); I(3, dim); I(4, act); F(5, lim); return ret_rc(env, dh_act_gate_rowsplit((const float*)in, (float*)o, T, dim, act, lim)); }
FN(js_argmax_workspace_bytes) { (void)info; return ret_num(env, (double)dh_argmax_workspace_bytes()); }
FN(js_argmax) {
  ARGS(7); P(0, lg); I(1, vocab); L(2, pad); F(3, cap); P(4, ws); P(5, tok); I(6, idx);
  return ret_rc(env, dh_argmax((const float*)lg, vocab, pad, cap, ws, (uint32_t*)tok, idx));
}
FN(js_sample_topk_workspace_bytes) { ARGS(2); I(0, vocab); I(1, k); return ret_num(env, (double)dh_sample_topk_workspace_bytes(vocab, k)); }
FN(js_sample_topk) {
  ARGS(10); P(0, lg); I(1, vocab); I(3, k); L(5, pad); F(6, cap); P(7, ws); P(8, tok); I(9, idx);
  double temperature, random_value;
  if (napi_get_value_double(env, a[2], &temperature) != napi_ok || napi_get_value_double(env, a[4], &random_value) != napi_ok) {
    napi_throw_type_error(env, NULL, "doppler_hip: number expected");
    return NULL;
  }
  return ret_rc(env, dh_sample_topk((const float*)lg, vocab, temperature, k, random_value, pad, cap, ws, (uint32_t*)tok, idx));
}
FN(js_cast_f32_to_f16) { ARGS(3); P(0, i); P(1, o); L(2, n); return ret_rc(env, dh_cast_f32_to_f16((const float*)i, o, n)); }
FN(js_cast_f16_to_f32) { ARGS(3); P(0, i); P(1, o); L(2, n); return ret_rc(env, dh_cast_f16_to_f32(i, (float*)o, n)); }
FN(js_matmul_rmsnorm_f32) {
  ARGS(11); P(0, x); P(1, W); I(2, tb); P(3, nw); I(4, nwdt); F(5, eps); I(6, off); P(7, res); P(8, out); I(9, N); I(10, K);
  return ret_rc(env, dh_matmul_rmsnorm_f32((const float*)x, (const float*)W, tb, nw, nwdt, eps, off, (const float*)res,
                                           (float*)out, N, K));
}
FN(js_matmul_rmsnorm_f16) {
  ARGS(11); P(0, x); P(1, W); I(2, tb); P(3, nw); I(4, nwdt); F(5, eps); I(6, off); P(7, res); P(8, out); I(9, N); I(10, K);
  return ret_rc(env, dh_matmul_rmsnorm_f16(x, W, tb, nw, nwdt, eps, off, res, out, N, K));
}
FN(js_check_finiteness) {
  ARGS(7); P(0, in); I(1, dt); L(2, n); P(3, st); I(4, layer); I(5, step); F(6, thr);
  return ret_rc(env, dh_check_finiteness(in, dt, n, (uint32_t*)st, (uint32_t)layer, (uint32_t)step, thr));
}

static napi_value module_init(napi_env env, napi_value exports) {
  static const struct { const char* name; napi_callback fn; } table[] = {
      {"graphBegin", js_graph_begin}, {"graphEnd", js_graph_end}, {"graphLaunch", js_graph_launch}, {"graphSetMaxPosition", js_graph_set_max_position}, {"graphPrepare", js_graph_prepare},
      {"graphDestroy", js_graph_destroy},
      {"init", js_init}, {"shutdown", js_shutdown}, {"sync", js_sync}, {"malloc", js_malloc}, {"free", js_free},
      {"upload", js_upload}, {"download", js_download}, {"copy", js_copy}, {"fillZero", js_fill_zero},
      {"eventCreate", js_event_create}, {"eventRecord", js_event_record}, {"eventElapsedMs", js_event_elapsed_ms},
      {"eventSynchronize", js_event_synchronize}, {"hostAlloc", js_host_alloc}, {"hostFree", js_host_free},
      {"downloadAsync", js_download_async},
      {"eventDestroy", js_event_destroy}, {"q4kDequant", js_q4k_dequant}, {"q4kMatmul", js_q4k_matmul},
      {"q4kFfnGateUp", js_q4k_ffn_gate_up}, {"f16wMatmul", js_f16w_matmul},
      {"q4kMatmulRmsnorm", js_q4k_matmul_rmsnorm}, {"q4kFfnGateUpRmsnorm", js_q4k_ffn_gate_up_rmsnorm},
      {"lmheadArgmaxWorkspaceBytes", js_lmhead_argmax_workspace_bytes}, {"lmheadArgmaxF16", js_lmhead_argmax_f16},
      {"lmheadArgmaxF16RMSNorm", js_lmhead_argmax_f16_rmsnorm},
      {"attnDecodeWorkspaceBytes", js_attn_decode_workspace_bytes}, {"attnDecode", js_attn_decode},
      {"attnDecodeStatic", js_attn_decode_static}, {"attnDecodeStaticMaxBytes", js_attn_decode_static_max_bytes},
      {"attnDecodeQkvSupported", js_attn_decode_qkv_supported}, {"attnDecodeQkv", js_attn_decode_qkv},
      {"attnDecodeKvLen", js_attn_decode_kvlen}, {"attnDecodeQkvKvLen", js_attn_decode_qkv_kvlen},
      {"attnDecodeQkvPartials", js_attn_decode_qkv_partials}, {"attnDecodeQkvKvLenPartials", js_attn_decode_qkv_kvlen_partials},
      {"chainStructSizes", js_chain_struct_sizes}, {"q4kGemvChain", js_q4k_gemv_chain}, {"q4kGemvChainAttn", js_q4k_gemv_chain_attn},
      {"q4kGemvChainAttnSupported", js_q4k_gemv_chain_attn_supported},
      {"attnPrefill", js_attn_prefill},
      {"rmsnorm", js_rmsnorm}, {"rmsnormQK", js_rmsnorm_qk}, {"rmsnormSandwichPair", js_rmsnorm_sandwich_pair},
      {"residualRmsnormPair", js_residual_rmsnorm_pair}, {"rope", js_rope}, {"ropeQK", js_rope_qk}, {"qkvNormRopeKvwrite", js_qkv_norm_rope_kvwrite},
      {"kvWriteF16", js_kv_write_f16}, {"residualAdd", js_residual_add}, {"biasAdd", js_bias_add}, {"splitQKV", js_split_qkv}, {"scale", js_scale}, {"gatherF16", js_gather_f16},
      {"actGate", js_act_gate}, {"actGateRowsplit", js_act_gate_rowsplit},
      {"argmaxWorkspaceBytes", js_argmax_workspace_bytes}, {"argmax", js_argmax},
      {"sampleTopkWorkspaceBytes", js_sample_topk_workspace_bytes}, {"sampleTopk", js_sample_topk},
      {"castF32ToF16", js_cast_f32_to_f16}, {"castF16ToF32", js_cast_f16_to_f32},
      {"matmulRmsnormF32", js_matmul_rmsnorm_f32}, {"matmulRmsnormF16", js_matmul_rmsnorm_f16}, {"checkFiniteness", js_check_finiteness},
  };
  for (size_t i = 0; i < sizeof(table) / sizeof(table[0]); i++) {
    napi_value fn;
    if (napi_create_function(env, table[i].name, NAPI_AUTO_LENGTH, table[i].fn, NULL, &fn) != napi_ok) return NULL;
    napi_set_named_property(env, exports, table[i].name, fn);
  }
  return exports;
}

NAPI_MODULE(NODE_GYP_MODULE_NAME, module_init)
