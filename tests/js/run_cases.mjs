// Runs op cases prepared by tests/test_gpu_js.py through the JavaScript host API
// (doppler_amd/js/kernel-selector.js -> Node-API addon -> libdopplerhip.so) and writes each
// result next to its inputs.  Usage: node tests/js/run_cases.mjs <case-dir>
import fs from 'fs';
import path from 'path';
import * as dh from '../../doppler_amd/js/kernel-selector.js';
import { HipTextDecoder } from '../../doppler_amd/js/pipeline/decode-step.js';
import { loadDecoderWeights, parseManifest } from '../../doppler_amd/js/loader/rdrr-loader.js';

const dir = process.argv[2];
const manifest = JSON.parse(fs.readFileSync(path.join(dir, 'manifest.json'), 'utf8'));

function load(name) {
  const b = fs.readFileSync(path.join(dir, name));
  return new Uint8Array(b.buffer, b.byteOffset, b.byteLength).slice();
}
function dev(name, label) {
  const bytes = load(name);
  const buf = dh.acquireBuffer(Math.max(bytes.byteLength, 4), undefined, label || name);
  dh.uploadData(buf, bytes);
  return buf;
}
function tensor(name, dtype, shape) {
  return dh.createTensor(dev(name), dtype, shape, name);
}
async function save(name, buffer, bytes) {
  const ab = await dh.readBuffer(buffer, bytes);
  fs.writeFileSync(path.join(dir, name), Buffer.from(ab));
}
async function expectThrow(results, label, pattern, fn) {
  try {
    await fn();
    results.errors.push({ label, ok: false, message: 'did not throw' });
  } catch (e) {
    results.errors.push({ label, ok: new RegExp(pattern).test(e.message), message: e.message });
  }
}

async function main() {
  const results = { cases: [], errors: [] };
  dh.initDevice(0);

  for (const c of manifest.cases) {
    const out = `${c.name}.out.bin`;
    if (c.op === 'dequant') {
      const t = await dh.runDequantQ4K(dh.createWeightBuffer(dev(c.W), 'q4k', 'row', [c.blocks, 256]), c.blocks);
      await save(out, t.buffer, c.blocks * 256 * 4);
    } else if (c.op === 'matmul') {
      const W = dh.createWeightBuffer(dev(c.W), c.wdtype, 'row', [c.N, c.K], c.name);
      const A = tensor(c.A, c.aDtype || 'f32', [c.M, c.K]);
      const opts = { outputDtype: c.outputDtype, alpha: c.alpha, role: 'test' };
      if (c.residual) opts.residualTensor = tensor(c.residual, 'f32', [c.M, c.N]);
      if (c.normWeight) {
        opts.normWeight = tensor(c.normWeight, 'f32', [c.K]);
        opts.rmsNormEps = c.rmsNormEps;
        opts.useFusedRmsnormWideTile = true;
      }
      const rec = c.record ? dh.createCommandRecorder('t') : null;
      const t = rec ? await dh.recordMatmul(rec, A, W, c.M, c.N, c.K, opts) : await dh.runMatmul(A, W, c.M, c.N, c.K, opts);
      if (rec) await rec.submitAndWait();
      await save(out, t.buffer, c.M * c.N * (c.outputDtype === 'f16' ? 2 : 4));
    } else if (c.op === 'fused_ffn') {
      const Wg = dh.createWeightBuffer(dev(c.Wg), 'q4k', 'row', [c.inter, c.hidden]);
      const Wu = dh.createWeightBuffer(dev(c.Wu), 'q4k', 'row', [c.inter, c.hidden]);
      const t = await dh.runFusedFFN(tensor(c.X, 'f32', [c.M, c.hidden]), Wg, Wu, c.hidden, c.inter,
        { batchSize: c.M, activation: c.activation, alpha: c.alpha, swigluLimit: c.swigluLimit });
      await save(out, t.buffer, c.M * c.inter * 4);
    } else if (c.op === 'fused_normed_ffn') {
      const Wg = dh.createWeightBuffer(dev(c.Wg), 'q4k', 'row', [c.inter, c.hidden]);
      const Wu = dh.createWeightBuffer(dev(c.Wu), 'q4k', 'row', [c.inter, c.hidden]);
      const t = await dh.runFusedNormedFFN(tensor(c.X, 'f32', [c.M, c.hidden]), tensor(c.normWeight, 'f32', [c.hidden]),
        c.eps, Wg, Wu, c.hidden, c.inter, { batchSize: c.M, activation: c.activation });
      await save(out, t.buffer, c.M * c.inter * 4);
    } else if (c.op === 'rmsnorm') {
      const opts = { batchSize: c.batch, hiddenSize: c.hidden, rmsNormWeightOffset: c.weightOffset };
      if (c.residual) opts.residual = tensor(c.residual, 'f32', [c.batch, c.hidden]);
      if (c.outputScale) opts.outputScale = c.outputScale;
      const t = await dh.runRMSNorm(tensor(c.x, 'f32', [c.batch, c.hidden]), tensor(c.w, 'f32', [c.hidden]), c.eps, opts);
      await save(out, t.buffer, c.batch * c.hidden * 4);
    } else if (c.op === 'rmsnorm_qk') {
      const q = tensor(c.q, 'f32', [c.T * c.heads, c.headDim]);
      const k = tensor(c.k, 'f32', [c.T * c.kvHeads, c.headDim]);
      if (!dh.canUseRMSNormQK(q, k) || dh.canUseRMSNormQK(q, q)) throw new Error('canUseRMSNormQK');
      const r = await dh.runRMSNormQK(q, k, tensor(c.qw, 'f32', [c.headDim]), tensor(c.kw, 'f32', [c.headDim]), c.eps,
        { numTokens: c.T, numHeads: c.heads, numKVHeads: c.kvHeads, headDim: c.headDim, rmsNormWeightOffset: true });
      await save(c.name + '.q.out.bin', r.q.buffer, c.T * c.heads * c.headDim * 4);
      await save(c.name + '.k.out.bin', r.k.buffer, c.T * c.kvHeads * c.headDim * 4);
    } else if (c.op === 'rmsnorm_pair') {
      const x = tensor(c.x, 'f32', [c.batch, c.hidden]);
      const r = tensor(c.r, 'f32', [c.batch, c.hidden]);
      const wa = tensor(c.wa, 'f32', [c.hidden]);
      const wb = tensor(c.wb, 'f32', [c.hidden]);
      const opts = { batchSize: c.batch, hiddenSize: c.hidden, rmsNormWeightOffset: true };
      const s = await dh.runSandwichRMSNormPair(x, r, wa, wb, c.eps, opts);
      await save(c.name + '.post.out.bin', s.postAttn.buffer, c.batch * c.hidden * 4);
      await save(c.name + '.pre.out.bin', s.ffnInput.buffer, c.batch * c.hidden * 4);
      const n = await dh.runResidualNextRMSNormPair(x, r, wa, c.eps, Object.assign({ outputScale: c.outputScale }, opts));
      await save(c.name + '.res.out.bin', n.residual.buffer, c.batch * c.hidden * 4);
      await save(c.name + '.next.out.bin', n.nextInput.buffer, c.batch * c.hidden * 4);
    } else if (c.op === 'rope') {
      const dt = c.dtype || 'f32';
      const x = tensor(c.x, dt, [c.seq, c.heads, c.headDim]);
      const t = await dh.runRoPE(x, tensor(c.cos, 'f32', [1]), tensor(c.sin, 'f32', [1]), c.seq,
        { numHeads: c.heads, headDim: c.headDim, startPos: c.startPos, interleaved: c.interleaved });
      if (t.buffer !== x.buffer || t.dtype !== dt) throw new Error('runRoPE must alias its input and keep its dtype');
      await save(out, t.buffer, c.seq * c.heads * c.headDim * (dt === 'f16' ? 2 : 4));
    } else if (c.op === 'rope_qk') {
      const q = tensor(c.q, 'f32', [c.seq, c.heads, c.headDim]);
      const k = tensor(c.k, 'f32', [c.seq, c.kvHeads, c.headDim]);
      if (!dh.canUseRoPEQK(q, k) || dh.canUseRoPEQK(q, q)) throw new Error('canUseRoPEQK');
      const r = await dh.runRoPEQK(q, k, tensor(c.cos, 'f32', [1]), tensor(c.sin, 'f32', [1]), c.seq,
        { numQHeads: c.heads, numKVHeads: c.kvHeads, headDim: c.headDim, startPos: c.startPos });
      if (r.q.buffer !== q.buffer || r.k.buffer !== k.buffer) throw new Error('runRoPEQK must alias its inputs');
      await save(c.name + '.q.out.bin', r.q.buffer, c.seq * c.heads * c.headDim * 4);
      await save(c.name + '.k.out.bin', r.k.buffer, c.seq * c.kvHeads * c.headDim * 4);
    } else if (c.op === 'split_plain') {
      const r = await dh.runSplitQKV(tensor(c.x, 'f32', [c.tokens, c.q + c.k + c.v]),
        { numTokens: c.tokens, qSize: c.q, kSize: c.k, vSize: c.v });
      await save(c.name + '.q.out.bin', r.Q.buffer, c.tokens * c.q * 4);
      await save(c.name + '.k.out.bin', r.K.buffer, c.tokens * c.k * 4);
      await save(c.name + '.v.out.bin', r.V.buffer, c.tokens * c.v * 4);
    } else if (c.op === 'bias_scale') {
      const x = tensor(c.x, 'f32', [c.tokens, c.dim]);
      const b = await dh.runBiasAdd(x, tensor(c.bias, 'f32', [2, c.dim]), c.tokens, c.dim, { biasOffset: c.dim * 4 });
      if (b.buffer !== x.buffer) throw new Error('runBiasAdd must alias its data');
      const s = await dh.runScale(b, c.scale);
      await save(c.name + '.bias.out.bin', b.buffer, c.tokens * c.dim * 4);
      await save(c.name + '.scale.out.bin', s.buffer, c.tokens * c.dim * 4);
    } else if (c.op === 'split_qkv') {
      const ck = dh.acquireBuffer(c.maxSeq * c.kvHeads * c.headDim * 2);
      const cv = dh.acquireBuffer(c.maxSeq * c.kvHeads * c.headDim * 2);
      const r = await dh.runSplitQKVRMSNormRoPEQK(tensor(c.qkv, 'f32', [c.T, (c.heads + 2 * c.kvHeads) * c.headDim]),
        tensor(c.qw, 'f32', [c.headDim]), tensor(c.kw, 'f32', [c.headDim]), tensor(c.cos, 'f32', [1]), tensor(c.sin, 'f32', [1]),
        c.eps, { numTokens: c.T, numHeads: c.heads, numKVHeads: c.kvHeads, headDim: c.headDim, qSize: c.heads * c.headDim,
          kSize: c.kvHeads * c.headDim, vSize: c.kvHeads * c.headDim, startPos: c.startPos,
          f16KVCacheWrite: { keysBuffer: ck, valuesBuffer: cv, dstOffset: c.startPos * c.kvHeads * c.headDim } });
      await save(out, r.Q.buffer, c.T * c.heads * c.headDim * 4);
      await save(`${c.name}.k.bin`, ck, c.maxSeq * c.kvHeads * c.headDim * 2);
      await save(`${c.name}.v.bin`, cv, c.maxSeq * c.kvHeads * c.headDim * 2);
    } else if (c.op === 'kv_write') {
      const ck = dh.acquireBuffer(c.cacheElems * 2);
      const cv = dh.acquireBuffer(c.cacheElems * 2);
      await dh.runKVCacheWriteF32ToF16(dev(c.k), dev(c.v), ck, cv, { srcOffset: c.srcOffset, dstOffset: c.dstOffset, elementCount: c.count });
      await save(out, ck, c.cacheElems * 2);
      await save(`${c.name}.v.bin`, cv, c.cacheElems * 2);
    } else if (c.op === 'attention') {
      const dt = c.dtype || 'f32';
      const t = await dh.runAttention(tensor(c.Q, dt, [c.heads, c.headDim]), tensor(c.K, 'f16', [c.kvLen, c.kvHeads, c.headDim]),
        tensor(c.V, 'f16', [c.kvLen, c.kvHeads, c.headDim]), null, c.heads, c.headDim,
        { seqLen: 1, kvLen: c.kvLen, numKVHeads: c.kvHeads, causal: true, startPos: c.kvLen - 1 });
      if (t.dtype !== dt) throw new Error(`runAttention with ${dt} Q must return ${dt}, got ${t.dtype}`);
      await save(out, t.buffer, c.heads * c.headDim * (dt === 'f16' ? 2 : 4));
    } else if (c.op === 'attention_kvlen_buffer') {
      // the key count comes from a device u32 (kvLenBuffer); kvLen only bounds it
      const lenBuf = dh.acquireBuffer(4);
      dh.uploadData(lenBuf, new Uint32Array([c.count]));
      const t = await dh.runAttention(tensor(c.Q, 'f32', [c.heads, c.headDim]), tensor(c.K, 'f16', [c.kvLen, c.kvHeads, c.headDim]),
        tensor(c.V, 'f16', [c.kvLen, c.kvHeads, c.headDim]), null, c.heads, c.headDim,
        { seqLen: 1, kvLen: c.kvLen, numKVHeads: c.kvHeads, causal: true, startPos: -1, kvLenBuffer: lenBuf });
      await save(out, t.buffer, c.heads * c.headDim * 4);
      let refused = false;
      try {
        await dh.runAttention(tensor(c.Q, 'f32', [c.heads, c.headDim]), tensor(c.K, 'f16', [c.kvLen, c.kvHeads, c.headDim]),
          tensor(c.V, 'f16', [c.kvLen, c.kvHeads, c.headDim]), null, c.heads, c.headDim,
          { seqLen: 2, kvLen: c.kvLen, numKVHeads: c.kvHeads, kvLenBuffer: lenBuf });
      } catch (error) {
        refused = /kvLenBuffer/.test(error.message);
      }
      if (!refused) throw new Error('prefill with kvLenBuffer should be refused by name');
    } else if (c.op === 'attention_from_qkv') {
      // cache pre-filled with history rows; the op appends the row of startPos itself
      const keys = tensor(c.K, 'f16', [c.maxSeq, c.kvHeads, c.headDim]);
      const values = tensor(c.V, 'f16', [c.maxSeq, c.kvHeads, c.headDim]);
      if (!dh.decodeAttentionFromQKVSupported(c.heads, c.kvHeads, c.headDim)) throw new Error('fused decode attention should serve this geometry');
      const t = await dh.runDecodeAttentionFromQKV(tensor(c.qkv, 'f32', [1, (c.heads + 2 * c.kvHeads) * c.headDim]),
        tensor(c.qw, 'f32', [c.headDim]), tensor(c.kw, 'f32', [c.headDim]), tensor(c.cos, 'f32', [1]), tensor(c.sin, 'f32', [1]),
        c.eps, keys, values, { numHeads: c.heads, numKVHeads: c.kvHeads, headDim: c.headDim, startPos: c.startPos });
      await save(out, t.buffer, c.heads * c.headDim * 4);
      await save(`${c.name}.k.bin`, keys.buffer, c.maxSeq * c.kvHeads * c.headDim * 2);
      await save(`${c.name}.v.bin`, values.buffer, c.maxSeq * c.kvHeads * c.headDim * 2);
    } else if (c.op === 'residual') {
      const t = await dh.runResidualAdd(tensor(c.a, 'f32', [c.n]), tensor(c.b, 'f32', [c.n]), c.n, { outputScale: c.outputScale });
      await save(out, t.buffer, c.n * 4);
    } else if (c.op === 'silu_rowsplit') {
      const t = await dh.runSiLURowSplit(tensor(c.x, 'f32', [c.T, 2 * c.dim]), { numTokens: c.T, dim: c.dim, activation: c.activation });
      await save(out, t.buffer, c.T * c.dim * 4);
    } else if (c.op === 'gated') {
      const fn = c.activation === 'silu' ? dh.runSiLU : dh.runGeLU;
      const t = await fn(tensor(c.up, 'f32', [c.n]), { size: c.n, gate: tensor(c.gate, 'f32', [c.n]) });
      await save(out, t.buffer, c.n * 4);
    } else if (c.op === 'gather') {
      const dt = c.dtype || 'f32';
      const t = await dh.runGather(dev(c.ids), dev(c.table), c.T, c.hidden, c.vocab, { embeddingDtype: 'f16', outputDtype: dt });
      if (t.dtype !== dt) throw new Error(`runGather must return ${dt}, got ${t.dtype}`);
      await save(out, t.buffer, c.T * c.hidden * (dt === 'f16' ? 2 : 4));
    } else if (c.op === 'argmax') {
      const tok = await dh.runArgmax(dev(c.logits), c.vocab, { padTokenId: c.padTokenId });
      fs.writeFileSync(path.join(dir, out), Buffer.from(new Uint32Array([tok]).buffer));
    } else if (c.op === 'lm_head') {
      const rec = dh.createCommandRecorder('lm');
      const E = dh.createWeightBuffer(dev(c.E), 'f16', 'row', [c.vocab, c.hidden]);
      const opts = { vocabSize: c.vocab, hiddenSize: c.hidden };
      if (c.normWeight) {
        if (!dh.lmHeadArgmaxNormFusable(c.hidden)) throw new Error('lmHeadArgmaxNormFusable');
        opts.normWeight = tensor(c.normWeight, 'f32', [c.hidden]);
        opts.rmsNormEps = c.rmsNormEps;
      }
      const buf = await dh.recordLmHeadArgmaxF16(rec, tensor(c.h, 'f32', [1, c.hidden]), E, opts);
      await rec.submitAndWait();
      await save(out, buf, 4);
    } else if (c.op === 'decoder') {
      const cfg = c.config;
      const weights = {
        layers: c.layers.map((l) => ({
          wqkv: load(l.wqkv), wo: load(l.wo), wgate: load(l.wgate), wup: load(l.wup), wdown: load(l.wdown),
          inputNorm: load(l.inputNorm), postAttnNorm: load(l.postAttnNorm), qNorm: load(l.qNorm), kNorm: load(l.kNorm),
        })),
        embed: load(c.embed), finalNorm: load(c.finalNorm), cos: load(c.cos), sin: load(c.sin),
      };
      const dec = new HipTextDecoder(cfg, weights);
      if (c.expectChained !== undefined) {
        results.errors.push({ label: `${c.name}-chained`, ok: dec.chainGemvs === c.expectChained, message: `chainGemvs=${dec.chainGemvs}` });
      }
      const tokens = [];
      let tok = c.prompt[0];
      for (let pos = 0; pos < c.prompt.length + c.steps; pos++) {
        const inp = pos < c.prompt.length ? c.prompt[pos] : tok;
        if (c.greedyFrom !== undefined && pos === c.greedyFrom) {
          // the rest of the tokens from the generation loop with staged readback, twice (the second call
          // reuses the pinned ring and overwrites the same KV rows with the same values)
          const n = c.prompt.length + c.steps - pos;
          const first = await dec.decodeGreedy(inp, pos, n);
          const again = await dec.decodeGreedy(inp, pos, n);
          results.errors.push({ label: `${c.name}-greedy-repeat`, ok: JSON.stringify(first) === JSON.stringify(again), message: JSON.stringify([first, again]) });
          tokens.push(...first);
          break;
        }
        if (c.graphFrom !== undefined && pos >= c.graphFrom && pos % 5 !== 4) {
          // replay of the captured step (captured at the first such position), an eager step now and then
          tok = await dec.decodeStepGraph(inp, pos);
        } else if (c.profileAt === pos) {
          // per-label HIP-event timings of one step (reference: createProfilingRecorder + resolveProfileTimings)
          const rec = dh.createProfilingRecorder('profiled_step');
          tok = await dec.decodeStep(inp, pos, { recorder: rec });
          results.profile = await rec.resolveProfileTimings();
          results.profileOps = rec.opCount;
        } else if (c.expectFinitenessAt === pos) {
          // the guard's bound is set below this model's activations: the step must throw and name layer and step
          let message = 'did not throw';
          try { await dec.decodeStep(inp, pos); } catch (e) { message = `${e.name}: ${e.message}`; }
          results.errors.push({ label: `${c.name}-guard`, ok: message === `FinitenessError: F16 bounds exceeded during generation (layer 0, step ${pos})`, message });
          break;
        } else {
          tok = await dec.decodeStep(inp, pos);
        }
        tokens.push(tok);
      }
      dec.releaseGraph();
      dec.releaseReadback();
      fs.writeFileSync(path.join(dir, out), Buffer.from(new Uint32Array(tokens).buffer));
    } else if (c.op === 'generate') {
      // RDRR artifact -> JS loader -> prefill path -> decode loop, greedy or sampled
      const { config, weights } = loadDecoderWeights(c.dir, c.maxSeq);
      const dec = new HipTextDecoder(config, weights);
      const tokens = await dec.generate(c.prompt, c.maxTokens, c.sampling || null);
      fs.writeFileSync(path.join(dir, out), Buffer.from(new Uint32Array(tokens).buffer));
    } else if (c.op === 'sample') {
      const tok = await dh.runGPUSample(dev(c.logits), c.vocab, { temperature: c.temperature, topK: c.topK, randomSeed: c.seed });
      fs.writeFileSync(path.join(dir, out), Buffer.from(new Uint32Array([tok]).buffer));
    } else if (c.op === 'rdrr_decoder') {
      // weights come from an RDRR artifact directory through the JS loader
      const { config, weights } = loadDecoderWeights(c.dir, c.maxSeq);
      const dec = new HipTextDecoder(config, weights);
      const tokens = [];
      let tok = c.prompt[0];
      for (let pos = 0; pos < c.prompt.length + c.steps; pos++) {
        tok = await dec.decodeStep(pos < c.prompt.length ? c.prompt[pos] : tok, pos);
        tokens.push(tok);
      }
      fs.writeFileSync(path.join(dir, out), Buffer.from(new Uint32Array(tokens).buffer));
    } else if (c.op === 'matmul_rmsnorm_fused') {
      const dt = c.dtype || 'f32';
      const opts = { N: c.N, K: c.K, eps: c.eps, transposeB: c.transposeB, rmsNormWeightOffset: c.weightOffset,
        residual: c.residual ? tensor(c.residual, dt, [1, c.N]) : null, label: 'test' };
      const x = tensor(c.x, dt, [1, c.K]);
      const W = dh.createWeightBuffer(dev(c.W), dt, 'row', c.transposeB ? [c.N, c.K] : [c.K, c.N], c.name);
      const nw = dev(c.normWeight);
      if (!dh.shouldUseFusedMatmulRMSNorm(1, c.N, c.K)) throw new Error('shouldUseFusedMatmulRMSNorm said no');
      const rec = c.record ? dh.createCommandRecorder('t') : null;
      const t = rec ? await dh.recordMatmulRMSNormFused(rec, x, W, nw, opts) : await dh.runMatmulRMSNormFused(x, W, nw, opts);
      if (rec) await rec.submitAndWait();
      await save(out, t.buffer, c.N * (dt === 'f16' ? 2 : 4));
    } else if (c.op === 'check_finiteness') {
      // one status buffer across the listed checks, in order: [input file, dtype, size, layer, step, threshold]
      const status = dh.createFinitenessStatusBuffer();
      const words = [];
      for (const k of c.checks) {
        dh.recordCheckFiniteness(null, tensor(k.input, k.dtype, [k.size]), k.size, status, k.layer, k.step, k.threshold === null ? undefined : k.threshold);
        words.push(...new Uint32Array(await dh.readBuffer(status, 16)));
      }
      fs.writeFileSync(path.join(dir, out), Buffer.from(new Uint32Array(words).buffer));
    } else {
      throw new Error(`unknown case op ${c.op}`);
    }
    results.cases.push(c.name);
  }

  // error behaviour (reference: synchronous validation -> thrown Error with an [Op] prefix)
  {
    const W = dh.createWeightBuffer(dh.acquireBuffer(8 * 144), 'q4k', 'row', [8, 256], 'w');
    const A = dh.createTensor(dh.acquireBuffer(1024), 'f32', [1, 256], 'a');
    await expectThrow(results, 'outputDtype', 'outputDtype is required', () => dh.runMatmul(A, W, 1, 8, 256, {}));
    await expectThrow(results, 'dims', 'Dimensions must be positive', () => dh.runMatmul(A, W, 0, 8, 256, { outputDtype: 'f32' }));
    await expectThrow(results, 'bsmall', 'B buffer too small', () => dh.runMatmul(A, W, 1, 9, 256, { outputDtype: 'f32' }));
    await expectThrow(results, 'asmall', 'A buffer too small', () => dh.runMatmul(A, W, 2, 8, 256, { outputDtype: 'f32' }));
    await expectThrow(results, 'bdtype', 'B dtype is required', () => dh.runMatmul(A, W.buffer, 1, 8, 256, { outputDtype: 'f32' }));
    await expectThrow(results, 'offsets', '256-byte aligned', () => dh.runMatmul(A, W, 1, 8, 256, { outputDtype: 'f32', aOffset: 4 }));
    await expectThrow(results, 'rope_qk', 'RoPE QK rotaryDim must be even', () => dh.runRoPEQK(A, dh.createTensor(dh.acquireBuffer(1024), 'f32', [1, 256], 'b'), A, A, 1, { numQHeads: 1, numKVHeads: 1, headDim: 64, rotaryDim: 31 }));
    await expectThrow(results, 'rope', 'rotaryDim must be even', () => dh.runRoPE(A, A, A, 1, { numHeads: 1, headDim: 64, rotaryDim: 31 }));
    await expectThrow(results, 'gather', 'embeddingDtype is required', () => dh.runGather(A.buffer, A.buffer, 1, 8, 8, {}));
    await expectThrow(results, 'kvwrite', 'smaller than requested range', () => dh.runKVCacheWriteF32ToF16(A.buffer, A.buffer, A.buffer, A.buffer, { elementCount: 100000 }));
    await expectThrow(results, 'attn', 'kvLayout', () => dh.runAttention(A, A, A, null, 2, 64, { kvLayout: 'paged' }));
    await expectThrow(results, 'rdrr-json', 'Failed to parse manifest JSON', async () => parseManifest('{'));
    await expectThrow(results, 'rdrr-shard', 'missing shard index', async () => parseManifest(JSON.stringify({
      shards: [{ filename: 'shard_00000.bin', size: 1024 }], tensors: { w: { offset: 0, size: 4, shape: [1], dtype: 'F32' } } })));
    await expectThrow(results, 'rdrr-size', 'should hold 144 bytes', async () => parseManifest(JSON.stringify({
      shards: [{ filename: 'shard_00000.bin', size: 1024 }], tensors: { w: { shard: 0, offset: 0, size: 100, shape: [1, 256], dtype: 'Q4_K_M' } } })));
    await expectThrow(results, 'fused-mr-tb', 'transposeB is required', () => dh.runMatmulRMSNormFused(A, A, A, { N: 4, K: 8, eps: 1e-6, rmsNormWeightOffset: false }));
    await expectThrow(results, 'fused-mr-n', 'exceeds maxMediumN=4096', () => dh.runMatmulRMSNormFused(A, A, A, { N: 4097, K: 8, eps: 1e-6, transposeB: true, rmsNormWeightOffset: false }));
    await expectThrow(results, 'fused-mr-nw', 'does not match hiddenSize=1024', () => dh.runMatmulRMSNormFused(A, A, A, { N: 1024, K: 8, eps: 1e-6, transposeB: true, rmsNormWeightOffset: false }));
    await expectThrow(results, 'f16a-norm', 'f16 activations are served', () => dh.runMatmul(dh.createTensor(A.buffer, 'f16', [1, 256]), W, 1, 8, 256, { outputDtype: 'f32', normWeight: A, rmsNormEps: 1e-6, useFusedRmsnormWideTile: true }));
    await expectThrow(results, 'finite-status', 'status buffer must hold', () => dh.recordCheckFiniteness(null, A, 4, dh.acquireBuffer(8)));
    if (dh.selectMatmulRMSNormFusedVariant(256, 'f32') !== 'small' || dh.selectMatmulRMSNormFusedVariant(1152, 'f16') !== 'medium_f16' ||
        dh.shouldUseFusedMatmulRMSNorm(2, 8, 8) || dh.shouldUseFusedMatmulRMSNorm(1, 8, 8193) || !dh.shouldUseFusedMatmulRMSNorm(1, 4096, 8192) ||
        dh.resolveFinitenessAbsThreshold(-1) !== 65500 || dh.resolveFinitenessAbsThreshold(50000) !== 50000 ||
        dh.shouldTriggerFinitenessValue(100) || !dh.shouldTriggerFinitenessValue(65501, 65500) || !dh.shouldTriggerFinitenessValue(NaN, 65500) ||
        dh.parseFinitenessStatusWords(new Uint32Array([42, 1, 3, 15, 0]), 1).metadata !== ' (layer 3, step 15)' ||
        dh.parseFinitenessStatusWords(new Uint32Array([0, 7, 9]), 0).triggered) {
      results.errors.push({ label: 'host-helpers', ok: false, message: 'a selection or finiteness helper disagrees with the reference tests' });
    } else {
      results.errors.push({ label: 'host-helpers', ok: true, message: '' });
    }
    await expectThrow(results, 'ffn', 'matching gate/up dtypes', () => dh.runFusedFFN(A, W, dh.createWeightBuffer(W.buffer, 'f16', 'row', [8, 256]), 256, 8, {}));
  }

  fs.writeFileSync(path.join(dir, 'results.json'), JSON.stringify(results));
  console.log(`ran ${results.cases.length} cases`);
}

main().catch((e) => {
  console.error(e && e.stack ? e.stack : e);
  process.exit(1);
});
