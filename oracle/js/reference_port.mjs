// TEST INFRASTRUCTURE, not part of the product: a single-threaded JavaScript restatement of the
// reference's CPU per-op references, used (a) to time "what the reference's own CPU path costs"
// on the benchmark host under Node, beside the HIP path, and (b) as a second, independent
// statement of the Q4_K arithmetic that tests compare with the C oracle.
//
// Follows (read as text, rewritten here):
//   Q4_K super-block decode   tests/kernels/reference/dequant.js:253-300 (dequantizeQ4_KBlockRef)
//   f16 -> f32                tests/kernels/reference/dequant.js:8-24
//   row-wise tensor decode    tests/kernels/reference/fused-ffn-q4k.js:24-40 (dequantQ4KRowsRef)
//   C = A . W^T, f64 sum      tests/kernels/browser/kernel-suite.js:152-166 (matmulRefRowMajorB)
//   gated FFN                 tests/kernels/reference/fused-ffn-q4k.js:42-73 (fusedFfnQ4KRef)
//   decode attention          tests/kernels/reference/attention.js:4-63 (attentionRef)
//
//   node reference_port.mjs time                 -> one JSON line of timings (ms)
//   node reference_port.mjs gemv in.bin out.bin  -> y = x . dequant(W)^T for a case read from in.bin
//
// in.bin: int32 M, N, K, then M*K f32 activations, then N*ceil(K/256)*144 weight bytes.
// out.bin: M*N f32.
import fs from 'fs';

const QK = 256, BLOCK_BYTES = 144;

function halfToFloat(bits) {
  const sign = (bits & 0x8000) ? -1 : 1;
  const exp = (bits >> 10) & 0x1f, frac = bits & 0x3ff;
  if (exp === 0) return sign * frac * Math.pow(2, -24);
  if (exp === 31) return frac ? NaN : sign * Infinity;
  return sign * (1 + frac / 1024) * Math.pow(2, exp - 15);
}

// Decodes one 144-byte super-block at byte offset `off` into out[o .. o+255].
function decodeBlock(bytes, off, out, o) {
  const d = halfToFloat(bytes[off] | (bytes[off + 1] << 8));
  const dmin = halfToFloat(bytes[off + 2] | (bytes[off + 3] << 8));
  const sc = new Array(8), mn = new Array(8);
  for (let i = 0; i < 4; i++) {
    sc[i] = bytes[off + 4 + i] & 63;
    mn[i] = bytes[off + 8 + i] & 63;
    sc[i + 4] = (bytes[off + 12 + i] & 15) | ((bytes[off + 4 + i] >> 6) << 4);
    mn[i + 4] = (bytes[off + 12 + i] >> 4) | ((bytes[off + 8 + i] >> 6) << 4);
  }
  for (let chunk = 0; chunk < 4; chunk++) {
    const sLo = Math.fround(d * sc[2 * chunk]), mLo = Math.fround(dmin * mn[2 * chunk]);
    const sHi = Math.fround(d * sc[2 * chunk + 1]), mHi = Math.fround(dmin * mn[2 * chunk + 1]);
    const q = off + 16 + 32 * chunk;
    for (let j = 0; j < 32; j++) {
      const b = bytes[q + j];
      out[o + 64 * chunk + j] = sLo * (b & 15) - mLo;            // stored to Float32Array: one rounding
      out[o + 64 * chunk + 32 + j] = sHi * (b >> 4) - mHi;
    }
  }
}

// W [N][K] in row layout -> Float32Array [N][K] (the padded tail of each row is dropped).
function decodeRows(bytes, N, K) {
  const nb = Math.ceil(K / QK);
  const out = new Float32Array(N * K), tmp = new Float32Array(QK);
  for (let n = 0; n < N; n++) {
    for (let b = 0; b < nb; b++) {
      decodeBlock(bytes, (n * nb + b) * BLOCK_BYTES, tmp, 0);
      const k0 = b * QK, len = Math.min(QK, K - k0);
      for (let k = 0; k < len; k++) out[n * K + k0 + k] = tmp[k];
    }
  }
  return out;
}

function matmulRowMajorB(A, W, M, N, K) {
  const C = new Float32Array(M * N);
  for (let m = 0; m < M; m++)
    for (let n = 0; n < N; n++) {
      let sum = 0;
      for (let k = 0; k < K; k++) sum += A[m * K + k] * W[n * K + k];
      C[m * N + n] = sum;
    }
  return C;
}

function geluTanh(x) {
  return 0.5 * x * (1 + Math.tanh(0.7978845608 * (x + 0.044715 * x * x * x)));
}

function gatedFfn(X, Wg, Wu, Wd, M, hidden, inter) {
  const g = matmulRowMajorB(X, Wg, M, inter, hidden), u = matmulRowMajorB(X, Wu, M, inter, hidden);
  const h = new Float32Array(M * inter);
  for (let i = 0; i < h.length; i++) h[i] = geluTanh(g[i]) * u[i];
  return matmulRowMajorB(h, Wd, M, hidden, inter);
}

// One query token; K and V [kvLen][Hkv][D] as f32 values of f16 numbers.
function attentionDecode(Q, Kc, Vc, H, Hkv, D, kvLen, scale) {
  const O = new Float32Array(H * D), scores = new Float64Array(kvLen);
  for (let h = 0; h < H; h++) {
    const kvh = Math.floor(h / (H / Hkv));
    let mx = -Infinity;
    for (let t = 0; t < kvLen; t++) {
      let s = 0;
      for (let d = 0; d < D; d++) s += Q[h * D + d] * Kc[(t * Hkv + kvh) * D + d];
      scores[t] = s * scale;
      if (scores[t] > mx) mx = scores[t];
    }
    let den = 0;
    for (let t = 0; t < kvLen; t++) { scores[t] = Math.exp(scores[t] - mx); den += scores[t]; }
    for (let d = 0; d < D; d++) {
      let acc = 0;
      for (let t = 0; t < kvLen; t++) acc += (scores[t] / den) * Vc[(t * Hkv + kvh) * D + d];
      O[h * D + d] = acc;
    }
  }
  return O;
}

// ---- seeded inputs for the timing mode (a 32-bit LCG; values only need the right ranges)
function makeRng(seed) {
  let s = seed >>> 0;
  return () => { s = (Math.imul(s, 1664525) + 1013904223) >>> 0; return s / 4294967296; };
}
function randomQ4K(N, K, rng) {
  const nb = Math.ceil(K / QK), bytes = new Uint8Array(N * nb * BLOCK_BYTES);
  for (let i = 0; i < bytes.length; i++) bytes[i] = (rng() * 256) | 0;
  for (let b = 0; b < N * nb; b++) {          // d, dmin around 0.01 (f16 0x2120 .. 0x213f)
    bytes[b * BLOCK_BYTES] = 0x20 + ((rng() * 32) | 0); bytes[b * BLOCK_BYTES + 1] = 0x21;
    bytes[b * BLOCK_BYTES + 2] = 0x20 + ((rng() * 32) | 0); bytes[b * BLOCK_BYTES + 3] = 0x21;
  }
  return bytes;
}
function randomF32(n, rng, scale) {
  const a = new Float32Array(n);
  for (let i = 0; i < n; i++) a[i] = (rng() + rng() + rng() + rng() - 2) * 1.7320508 * scale;   // ~N(0, scale^2)
  return a;
}
function ms(fn) {
  const t0 = process.hrtime.bigint();
  const r = fn();
  return [Number(process.hrtime.bigint() - t0) / 1e6, r];
}

function timeAll() {
  const rng = makeRng(12345);
  const out = { node: process.version, threads: 1 };
  let sink = 0;
  {   // config 0: one 640 -> 2048 GEMV (decode + dot, as the reference's matmul_q4k case does)
    const W = randomQ4K(2048, 640, rng), x = randomF32(640, rng, 1);
    const [t, y] = ms(() => matmulRowMajorB(x, decodeRows(W, 2048, 640), 1, 2048, 640));
    out.cfg0_gemv_ms = +t.toFixed(3); sink += y[0];
  }
  {   // config 1: the seven linear layers of a hidden-1024 block, M in {1, 2, 4, 8}
    const shapes = [[2048, 1024], [1024, 1024], [1024, 1024], [1024, 2048], [3072, 1024], [3072, 1024], [1024, 3072]];
    const Ws = shapes.map(([N, K]) => randomQ4K(N, K, rng));
    out.cfg1_block_ms = {};
    for (const M of [1, 2, 4, 8]) {
      let total = 0;
      shapes.forEach(([N, K], i) => {
        const A = randomF32(M * K, rng, 1);
        const [t, y] = ms(() => matmulRowMajorB(A, decodeRows(Ws[i], N, K), M, N, K));
        total += t; sink += y[0];
      });
      out.cfg1_block_ms['M' + M] = +total.toFixed(2);
    }
  }
  {   // config 2, reduced to 8 of the 512 rows: gelu-gated FFN 1152 -> 6912 -> 1152
    const M = 8, hidden = 1152, inter = 6912;
    const Wg = randomQ4K(inter, hidden, rng), Wu = randomQ4K(inter, hidden, rng), Wd = randomQ4K(hidden, inter, rng);
    const X = randomF32(M * hidden, rng, 0.05);
    const [t, y] = ms(() => gatedFfn(X, decodeRows(Wg, inter, hidden), decodeRows(Wu, inter, hidden),
                                     decodeRows(Wd, hidden, inter), M, hidden, inter));
    out.cfg2_ffn_8_of_512_rows_ms = +t.toFixed(2); sink += y[0];
    out.cfg2_flop = 2 * M * hidden * inter * 3;
  }
  {   // config 3 at context 512: 16 query heads over 8 kv heads of 128
    const H = 16, Hkv = 8, D = 128, ctx = 512;
    const Q = randomF32(H * D, rng, 0.088), Kc = randomF32(ctx * Hkv * D, rng, 0.088), Vc = randomF32(ctx * Hkv * D, rng, 0.088);
    const [t, o] = ms(() => attentionDecode(Q, Kc, Vc, H, Hkv, D, ctx, 1 / Math.sqrt(D)));
    out.cfg3_attn_ctx512_ms = +t.toFixed(3); sink += o[0];
  }
  out.checksum = +sink.toFixed(6);
  console.log(JSON.stringify(out));
}

function gemvFile(inPath, outPath) {
  const buf = fs.readFileSync(inPath);
  const hdr = new Int32Array(buf.buffer, buf.byteOffset, 3);
  const [M, N, K] = hdr;
  const A = new Float32Array(buf.buffer.slice(buf.byteOffset + 12, buf.byteOffset + 12 + 4 * M * K));
  const W = new Uint8Array(buf.buffer, buf.byteOffset + 12 + 4 * M * K);
  const C = matmulRowMajorB(A, decodeRows(W, N, K), M, N, K);
  fs.writeFileSync(outPath, Buffer.from(C.buffer));
}

const mode = process.argv[2];
if (mode === 'time') timeAll();
else if (mode === 'gemv') gemvFile(process.argv[3], process.argv[4]);
else { console.error('usage: node reference_port.mjs time | gemv in.bin out.bin'); process.exit(2); }
