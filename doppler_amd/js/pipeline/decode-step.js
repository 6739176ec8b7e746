// Greedy decode loop over the HIP op API: the shape of the reference's decodeStep
// (src/inference/pipelines/text/generator-steps.js:588-820) for a Qwen3-class Q4_K model.
// One CommandRecorder per token, every op recorded in execution-graph order
// (src/config/conversion/qwen3/qwen-3-embedding-0-6b-q4k-ehf16-af32.json `execution.decode`),
// one 4-byte readback per token.
import {
  createTensor, createWeightBuffer, acquireBuffer, releaseBuffer, uploadData, readBufferSlice,
  createCommandRecorder, recordGather, recordRMSNorm, recordMatmul, recordSplitQKVRMSNormRoPEQK,
  recordAttention, recordFusedNormedFFN, recordFusedFFN, recordLmHeadArgmaxF16, lmHeadArgmaxNormFusable, recordGPUSample,
  recordDecodeAttentionFromQKV, decodeAttentionFromQKVSupported,
  recordLayerChain, recordDecodeAttentionPartials, layerChainSupported, layerChainMergesAttention,
  recordCheckFiniteness, parseFinitenessStatusWords, resolveFinitenessAbsThreshold, FINITENESS_STATUS_BYTES,
} from '../kernel-selector.js';
import { getNative } from '../native.js';

// A window of a device buffer starting `offset` bytes in (no ownership: never released).
function bufferWindow(buffer, offset, size) {
  return { ptr: buffer.ptr + BigInt(offset), size, capacity: size, label: buffer.label };
}

// An activation left the f16 range (or the configured bound) during a decode step
// (reference: src/inference/pipelines/text/generator-steps.js:164-169).
export class FinitenessError extends Error {
  constructor(message) {
    super(message);
    this.name = 'FinitenessError';
  }
}

function upload(bytes, label) {
  const buf = acquireBuffer(bytes.byteLength, undefined, label);
  uploadData(buf, bytes);
  return buf;
}

// decodeGreedy: tokens in flight between the device and the host (ring slots), and the events that mark
// their copies
const TOKEN_RING = 64;
const READ_EVENTS = 4;

export class HipTextDecoder {
  // config: {layers, hidden, inter, heads, kvHeads, headDim, vocab, eps, maxSeq}
  //   finitenessGuard (default false): check every layer's output against finitenessAbsThreshold
  //   (one more launch per layer) and read the status words back beside the token, as the
  //   reference does for f16 activations (layer.js:1237-1252, generator-steps.js:786-798, :837-843)
  // weights: {layers: [{wqkv, wo, wgate, wup, wdown (Uint8Array Q4_K), inputNorm, postAttnNorm,
  //           qNorm, kNorm (Float32Array)}], embed (Uint16Array f16 bits), finalNorm, cos, sin}
  constructor(config, weights) {
    this.config = config;
    const c = config;
    this.qSize = c.heads * c.headDim;
    this.kSize = c.kvHeads * c.headDim;
    this.layers = weights.layers.map((l, i) => ({
      wqkv: createWeightBuffer(upload(l.wqkv, `L${i}.qkv`), 'q4k', 'row', [this.qSize + 2 * this.kSize, c.hidden], `L${i}.qkv`),
      wo: createWeightBuffer(upload(l.wo, `L${i}.o`), 'q4k', 'row', [c.hidden, this.qSize], `L${i}.o`),
      wgate: createWeightBuffer(upload(l.wgate, `L${i}.gate`), 'q4k', 'row', [c.inter, c.hidden], `L${i}.gate`),
      wup: createWeightBuffer(upload(l.wup, `L${i}.up`), 'q4k', 'row', [c.inter, c.hidden], `L${i}.up`),
      wdown: createWeightBuffer(upload(l.wdown, `L${i}.down`), 'q4k', 'row', [c.hidden, c.inter], `L${i}.down`),
      inputNorm: createTensor(upload(l.inputNorm), 'f32', [c.hidden], 'input_norm'),
      postAttnNorm: createTensor(upload(l.postAttnNorm), 'f32', [c.hidden], 'post_attn_norm'),
      qNorm: createTensor(upload(l.qNorm), 'f32', [c.headDim], 'q_norm'),
      kNorm: createTensor(upload(l.kNorm), 'f32', [c.headDim], 'k_norm'),
      cacheK: createTensor(acquireBuffer(c.maxSeq * this.kSize * 2, undefined, 'kv_k'), 'f16', [c.maxSeq, c.kvHeads, c.headDim], 'kv_k'),
      cacheV: createTensor(acquireBuffer(c.maxSeq * this.kSize * 2, undefined, 'kv_v'), 'f16', [c.maxSeq, c.kvHeads, c.headDim], 'kv_v'),
    }));
    this.embed = createWeightBuffer(upload(weights.embed, 'embed'), 'f16', 'row', [c.vocab, c.hidden], 'embed');
    this.finalNorm = createTensor(upload(weights.finalNorm), 'f32', [c.hidden], 'final_norm');
    this.cos = createTensor(upload(weights.cos), 'f32', [c.maxSeq, c.headDim / 2], 'rope_cos');
    this.sin = createTensor(upload(weights.sin), 'f32', [c.maxSeq, c.headDim / 2], 'rope_sin');
    // decode steps: q/k norm, RoPE and the KV append run inside the attention kernel when the head
    // geometry allows it (one launch fewer per layer)
    this.fuseQkvAttention = config.fuseQkvAttention !== false &&
      decodeAttentionFromQKVSupported(c.heads, c.kvHeads, c.headDim, c.headDim, false);
    // ... and the products between two attentions go out as one chained launch that also merges the
    // attention's key splits (two launches per layer), where the shapes are served and the guard is off
    this.chainGemvs = config.chainGemvs !== false && this.fuseQkvAttention && config.finitenessGuard !== true &&
      layerChainSupported(c.hidden, c.inter, this.qSize) && layerChainMergesAttention(c.heads, c.kvHeads, c.headDim, c.maxSeq);
    this.ids = acquireBuffer(16, undefined, 'token_ids');
    // [token, status, layer, step, pad]: the staging layout of the reference's guarded readback
    this.tokenOut = acquireBuffer(4 + FINITENESS_STATUS_BYTES, undefined, 'sampled_token');
    this.finitenessGuard = config.finitenessGuard === true;
    this.finitenessAbsThreshold = resolveFinitenessAbsThreshold(config.finitenessAbsThreshold);
    this.finitenessStatus = bufferWindow(this.tokenOut, 4, FINITENESS_STATUS_BYTES);
    this.logits = null;
    this.readback = null;
  }

  // Final RMSNorm + LM head + argmax of one hidden row: one launch with the norm inside the LM head kernel
  // where the hidden size allows it, else the norm as a launch of its own in front.
  async recordNormedLmHead(recorder, temps, hiddenRow, tokenOut, tokenIndex, logitsOutput) {
    const c = this.config;
    const opts = { vocabSize: c.vocab, hiddenSize: c.hidden, outputBuffer: tokenOut, outputIndex: tokenIndex, logitsOutput };
    if (lmHeadArgmaxNormFusable(c.hidden)) {
      await recordLmHeadArgmaxF16(recorder, hiddenRow, this.embed, Object.assign({ normWeight: this.finalNorm, rmsNormEps: c.eps }, opts));
      return;
    }
    const normed = await recordRMSNorm(recorder, hiddenRow, this.finalNorm, c.eps, { batchSize: 1, hiddenSize: c.hidden });
    temps.push(normed.buffer);
    await recordLmHeadArgmaxF16(recorder, normed, this.embed, opts);
  }

  // Final RMSNorm + LM head for one hidden row; greedy, or top-k temperature sampling when
  // `sampling` = {temperature, topK, randomSeed} is given (the logits then go through memory).
  async recordHead(recorder, temps, hiddenRow, sampling, tokenOut = this.tokenOut, tokenIndex = 0) {
    const c = this.config;
    if (sampling && !this.logits) this.logits = acquireBuffer(c.vocab * 4, undefined, 'logits');
    await this.recordNormedLmHead(recorder, temps, hiddenRow, tokenOut, tokenIndex, sampling ? this.logits : null);
    if (sampling) {
      await recordGPUSample(recorder, this.logits, c.vocab, Object.assign({ outputBuffer: tokenOut, outputIndex: tokenIndex }, sampling));
    }
  }

  // Pushes prompt tokens through the batched path (prefill GEMMs + prefill attention), `chunk`
  // tokens per pass, writing KV rows startPos.. ; returns the token after the last prompt token.
  // Mirrors the reference's prefill (src/inference/pipelines/text/generator.js) on the HIP ops.
  async prefill(tokens, startPos = 0, options = {}) {
    const c = this.config;
    const chunk = Math.max(1, Math.min(options.chunk || 2048, tokens.length));
    if (tokens.length === 0 || startPos + tokens.length > c.maxSeq) {
      throw new Error(`[prefill] ${tokens.length} tokens at ${startPos} do not fit maxSeq=${c.maxSeq}`);
    }
    const recorder = createCommandRecorder('prefill');
    const temps = [];
    const temp = (t) => { temps.push(t.buffer); return t; };
    const ids = acquireBuffer(chunk * 4, undefined, 'prefill_ids');
    temps.push(ids);
    let x = null, T = 0;
    for (let c0 = 0; c0 < tokens.length; c0 += chunk) {
      const part = tokens.slice(c0, c0 + chunk);
      T = part.length;
      const pos = startPos + c0;
      uploadData(ids, new Uint32Array(part));
      x = temp(await recordGather(recorder, ids, this.embed, T, c.hidden, c.vocab, { embeddingDtype: 'f16', outputDtype: 'f32' }));
      for (let li = 0; li < this.layers.length; li++) {
        const l = this.layers[li];
        // the input RMSNorm runs inside the product (GEMV prologue below 16 tokens, the GEMM's activation
        // packing from 16 on) unless the model asks for separate norm launches
        const fusedNorm = c.fuseNorm !== false;
        let qkv;
        if (fusedNorm) {
          qkv = temp(await recordMatmul(recorder, x, l.wqkv, T, this.qSize + 2 * this.kSize, c.hidden,
            { outputDtype: 'f32', role: 'qkv_proj', layerIdx: li,
              normWeight: l.inputNorm, rmsNormEps: c.eps, useFusedRmsnormWideTile: true }));
        } else {
          const normed = temp(await recordRMSNorm(recorder, x, l.inputNorm, c.eps, { batchSize: T, hiddenSize: c.hidden }));
          qkv = temp(await recordMatmul(recorder, normed, l.wqkv, T, this.qSize + 2 * this.kSize, c.hidden,
            { outputDtype: 'f32', role: 'qkv_proj', layerIdx: li }));
        }
        const split = await recordSplitQKVRMSNormRoPEQK(recorder, qkv, l.qNorm, l.kNorm, this.cos, this.sin, c.eps, {
          numTokens: T, numHeads: c.heads, numKVHeads: c.kvHeads, headDim: c.headDim,
          qSize: this.qSize, kSize: this.kSize, vSize: this.kSize, startPos: pos,
          f16KVCacheWrite: { keysBuffer: l.cacheK.buffer, valuesBuffer: l.cacheV.buffer, dstOffset: pos * this.kSize },
        });
        temp(split.Q);
        const attn = temp(await recordAttention(recorder, split.Q, l.cacheK, l.cacheV, null, c.heads, c.headDim, {
          seqLen: T, kvLen: pos + T, numKVHeads: c.kvHeads, causal: true, startPos: pos, layerIdx: li,
        }));
        const attnFlat = createTensor(attn.buffer, 'f32', [T, this.qSize], 'attn_flat');
        const x2 = temp(await recordMatmul(recorder, attnFlat, l.wo, T, c.hidden, this.qSize,
          { outputDtype: 'f32', role: 'o_proj', layerIdx: li, residualTensor: x }));
        let act;
        if (fusedNorm) {
          act = temp(await recordFusedNormedFFN(recorder, x2, l.postAttnNorm, c.eps, l.wgate, l.wup, c.hidden, c.inter,
            { batchSize: T, activation: 'silu' }));
        } else {
          const normed2 = temp(await recordRMSNorm(recorder, x2, l.postAttnNorm, c.eps, { batchSize: T, hiddenSize: c.hidden }));
          act = temp(await recordFusedFFN(recorder, normed2, l.wgate, l.wup, c.hidden, c.inter,
            { batchSize: T, activation: 'silu' }));
        }
        x = temp(await recordMatmul(recorder, act, l.wdown, T, c.hidden, c.inter,
          { outputDtype: 'f32', role: 'down_proj', layerIdx: li, residualTensor: x2 }));
      }
    }
    const lastRow = createTensor(bufferWindow(x.buffer, (T - 1) * c.hidden * 4, c.hidden * 4), 'f32', [1, c.hidden], 'last_hidden');
    await this.recordHead(recorder, temps, lastRow, options.sampling || null);
    for (const b of temps) recorder.trackTemporaryBuffer(b);
    recorder.submit();
    const bytes = await readBufferSlice(this.tokenOut, 0, 4);
    return new Uint32Array(bytes)[0];
  }

  // prefill + decode loop: returns the generated token ids.  sampling = {temperature, topK, seed}
  // draws token i with randomSeed seed + i (greedy when absent), as the reference's generator
  // advances its seed per step.
  async generate(promptTokens, maxTokens, sampling = null) {
    const draw = (i) => (sampling ? { temperature: sampling.temperature, topK: sampling.topK, randomSeed: sampling.seed + i } : null);
    const out = [];
    let tok = await this.prefill(promptTokens, 0, { sampling: draw(0) });
    out.push(tok);
    for (let i = 1; i < maxTokens; i++) {
      tok = await this.decodeStep(tok, promptTokens.length + i - 1, { sampling: draw(i) });
      out.push(tok);
    }
    return out;
  }

  // Records the ops of one decode step for the token id in this.ids at position `pos`; the new
  // token id goes to this.tokenOut.  Temporaries are pushed onto `temps`.
  // options.idsBuffer: the input token id is read from this device word instead; options.tokenOutBuffer /
  // tokenOutIndex: the new token goes to that word of that buffer instead.
  async recordDecodeStep(recorder, temps, pos, options = {}) {
    const c = this.config;
    if (!(pos >= 0 && pos < c.maxSeq)) {
      // the ops take no cache capacity: a position past the caches would write K/V out of bounds
      throw new Error(`[decodeStep] position ${pos} is outside the KV cache (maxSeq=${c.maxSeq})`);
    }
    const temp = (t) => { temps.push(t.buffer); return t; };
    const tokenOut = options.tokenOutBuffer || this.tokenOut, tokenIndex = options.tokenOutIndex || 0;
    let x = temp(await recordGather(recorder, options.idsBuffer || this.ids, this.embed, 1, c.hidden, c.vocab,
      { embeddingDtype: 'f16', outputDtype: 'f32' }));
    if (this.chainGemvs) {
      x = await this.recordChainedLayers(recorder, temps, x, pos, options);
    } else for (let li = 0; li < this.layers.length; li++) {
      const l = this.layers[li];
      // input RMSNorm runs in the prologue of the stacked q/k/v projection
      const qkv = temp(await recordMatmul(recorder, x, l.wqkv, 1, this.qSize + 2 * this.kSize, c.hidden,
        { outputDtype: 'f32', role: 'qkv_proj', layerIdx: li,
          normWeight: l.inputNorm, rmsNormEps: c.eps, useFusedRmsnormWideTile: true }));
      let attn;
      if (this.fuseQkvAttention) {
        attn = temp(await recordDecodeAttentionFromQKV(recorder, qkv, l.qNorm, l.kNorm, this.cos, this.sin, c.eps,
          l.cacheK, l.cacheV, { numHeads: c.heads, numKVHeads: c.kvHeads, headDim: c.headDim, startPos: pos, layerIdx: li,
            // a captured step reads the key count from the word behind the token id, so a replay needs no patching
            kvLenBuffer: options.deviceKvLen ? bufferWindow(this.ids, 4, 4) : null, maxKvLen: c.maxSeq }));
      } else {
        const split = await recordSplitQKVRMSNormRoPEQK(recorder, qkv, l.qNorm, l.kNorm, this.cos, this.sin, c.eps, {
          numTokens: 1, numHeads: c.heads, numKVHeads: c.kvHeads, headDim: c.headDim,
          qSize: this.qSize, kSize: this.kSize, vSize: this.kSize, startPos: pos,
          f16KVCacheWrite: { keysBuffer: l.cacheK.buffer, valuesBuffer: l.cacheV.buffer, dstOffset: pos * this.kSize },
        });
        temp(split.Q);
        attn = temp(await recordAttention(recorder, split.Q, l.cacheK, l.cacheV, null, c.heads, c.headDim, {
          seqLen: 1, kvLen: pos + 1, numKVHeads: c.kvHeads, causal: true, startPos: pos, layerIdx: li,
        }));
      }
      const attnFlat = createTensor(attn.buffer, 'f32', [1, this.qSize], 'attn_flat');
      const x2 = temp(await recordMatmul(recorder, attnFlat, l.wo, 1, c.hidden, this.qSize,
        { outputDtype: 'f32', role: 'o_proj', layerIdx: li, residualTensor: x }));
      const act = temp(await recordFusedNormedFFN(recorder, x2, l.postAttnNorm, c.eps, l.wgate, l.wup, c.hidden, c.inter,
        { batchSize: 1, activation: 'silu' }));
      x = temp(await recordMatmul(recorder, act, l.wdown, 1, c.hidden, c.inter,
        { outputDtype: 'f32', role: 'down_proj', layerIdx: li, residualTensor: x2 }));
      if (this.finitenessGuard) {
        recordCheckFiniteness(recorder, x, c.hidden, this.finitenessStatus, li, pos, this.finitenessAbsThreshold);
      }
    }
    if (options.sampling) {
      await this.recordHead(recorder, temps, x, options.sampling, tokenOut, tokenIndex);
    } else {
      await this.recordNormedLmHead(recorder, temps, x, tokenOut, tokenIndex, options.logitsOutput || null);
    }
  }

  // The layers of a decode step at two launches each: the attention's split kernel, then one chained
  // launch that merges the splits and runs o + residual, RMSNorm + gate/up + SiLU, down + residual and
  // the next layer's RMSNorm + q/k/v.  Returns the last layer's output row.
  async recordChainedLayers(recorder, temps, x, pos, options) {
    const c = this.config;
    const qkvSize = this.qSize + 2 * this.kSize;
    const f32 = (n, label) => { const b = acquireBuffer(n * 4, undefined, label); temps.push(b); return b; };
    const l0 = this.layers[0];
    let qkv = await recordMatmul(recorder, x, l0.wqkv, 1, qkvSize, c.hidden,
      { outputDtype: 'f32', role: 'qkv_proj', layerIdx: 0, normWeight: l0.inputNorm, rmsNormEps: c.eps, useFusedRmsnormWideTile: true });
    temps.push(qkv.buffer);
    let xb = x.buffer;
    for (let li = 0; li < this.layers.length; li++) {
      const l = this.layers[li];
      const next = li + 1 < this.layers.length ? this.layers[li + 1] : null;
      const attention = recordDecodeAttentionPartials(recorder, qkv, l.qNorm, l.kNorm, this.cos, this.sin, c.eps, l.cacheK, l.cacheV, {
        numHeads: c.heads, numKVHeads: c.kvHeads, headDim: c.headDim, startPos: pos,
        kvLenBuffer: options.deviceKvLen ? bufferWindow(this.ids, 4, 4) : null, maxKvLen: c.maxSeq,
      });
      temps.push(attention.workspace);
      const x2 = f32(c.hidden, 'attn_output'), act = f32(c.inter, 'ffn_act'), xOut = f32(c.hidden, 'layer_output');
      const phases = [
        { weight: l.wo, output: x2, residual: xb, N: c.hidden, K: this.qSize },
        { weight: l.wgate, weight2: l.wup, output: act, normWeight: l.postAttnNorm, N: c.inter, K: c.hidden, activation: 'silu', rmsNormEps: c.eps },
        { weight: l.wdown, output: xOut, residual: x2, N: c.hidden, K: c.inter },
      ];
      let qkvNext = null;
      if (next) {
        qkvNext = f32(qkvSize, 'qkv');
        phases.push({ weight: next.wqkv, output: qkvNext, normWeight: next.inputNorm, N: qkvSize, K: c.hidden, rmsNormEps: c.eps });
      }
      recordLayerChain(recorder, null, phases, attention);
      xb = xOut;
      if (next) qkv = createTensor(qkvNext, 'f32', [1, qkvSize], 'qkv');
    }
    return createTensor(xb, 'f32', [1, c.hidden], 'layer_output');
  }

  // Returns the greedy token for `token` at position `pos` (KV rows 0..pos-1 present).
  // options.recorder: a recorder of the caller's (e.g. a profiling one) instead of a fresh one.
  async decodeStep(token, pos, options = {}) {
    const recorder = options.recorder || createCommandRecorder('decode');
    const temps = [];
    uploadData(this.ids, new Uint32Array([token]));
    if (this.finitenessGuard) getNative().fillZero(this.tokenOut.ptr, 4, FINITENESS_STATUS_BYTES);
    await this.recordDecodeStep(recorder, temps, pos, options);
    for (const b of temps) recorder.trackTemporaryBuffer(b);
    recorder.submit();
    // the only device->host crossing: the token, with the guard's status words beside it
    const bytes = await readBufferSlice(this.tokenOut, 0, this.finitenessGuard ? 4 + FINITENESS_STATUS_BYTES : 4);
    const words = new Uint32Array(bytes);
    if (this.finitenessGuard) {
      const status = parseFinitenessStatusWords(words, 1);
      if (status.triggered) throw new FinitenessError(`F16 bounds exceeded during generation${status.metadata}`);
    }
    return words[0];
  }

  // n greedy steps starting with `token` at position `pos`; returns the n new token ids.  Every step's
  // token is read back (4 bytes per step, as in decodeStep), but one step late: step k + 1 takes its input
  // token from device memory and is enqueued before the host waits for token k, whose copy into pinned
  // memory was enqueued behind step k, so the GPU never waits for the host between steps (the reference
  // stages its token readbacks through a ring the same way, src/inference/decode-ring.js:141-177).  A
  // caller with a stop condition checks the tokens as they come and drops the one step in flight.
  async decodeGreedy(token, pos, n) {
    if (n <= 0) return [];
    if (this.finitenessGuard) {
      const guarded = [];
      for (let k = 0; k < n; k++) {
        token = await this.decodeStep(token, pos + k);
        guarded.push(token);
      }
      return guarded;
    }
    const native = getNative();
    if (!this.readback) {
      const host = native.hostAlloc(4 * TOKEN_RING);
      const events = [];
      for (let i = 0; i < READ_EVENTS; i++) events.push(native.eventCreate());
      this.readback = { host, tokens: new Uint32Array(host.view), events, ring: acquireBuffer(4 * TOKEN_RING, undefined, 'token_ring') };
    }
    const rb = this.readback;
    const enqueueStep = async (k) => {
      const recorder = createCommandRecorder('decode');
      const temps = [];
      const slot = k % TOKEN_RING;
      const options = { tokenOutBuffer: rb.ring, tokenOutIndex: slot };
      if (k > 0) options.idsBuffer = bufferWindow(rb.ring, 4 * ((k - 1) % TOKEN_RING), 4);
      await this.recordDecodeStep(recorder, temps, pos + k, options);
      for (const b of temps) recorder.trackTemporaryBuffer(b);
      recorder.submit();
      native.downloadAsync(rb.host.ptr, 4 * slot, rb.ring.ptr, 4 * slot, 4);
      native.eventRecord(rb.events[k % READ_EVENTS]);
    };
    const waitToken = (k) => {
      native.eventSynchronize(rb.events[k % READ_EVENTS]);
      return rb.tokens[k % TOKEN_RING];
    };
    uploadData(this.ids, new Uint32Array([token]));
    await enqueueStep(0);
    const out = [];
    for (let k = 1; k < n; k++) {
      await enqueueStep(k);
      out.push(waitToken(k - 1));
    }
    out.push(waitToken(n - 1));
    return out;
  }

  // Frees the pinned staging memory, the device ring and the events decodeGreedy made.
  releaseReadback() {
    if (this.readback) {
      const native = getNative();
      native.sync();
      for (const ev of this.readback.events) native.eventDestroy(ev);
      this.readback.tokens = null;
      native.hostFree(this.readback.host.ptr);
      releaseBuffer(this.readback.ring);
      this.readback = null;
    }
  }

  // Captures the decode step into a HIP graph, the counterpart of the reference's
  // one-submit-per-step recorder (generator-steps.js:605,814).  The step runs once normally first
  // (every kernel's one-time set-up then lies outside the capture); the buffers the captured step
  // uses stay allocated for the graph's life.
  async captureDecodeStep(token, pos) {
    if (!this.fuseQkvAttention) throw new Error('[captureDecodeStep] serves the fused-attention step');
    const c = this.config;
    const first = await this.decodeStep(token, pos);
    uploadData(this.ids, new Uint32Array([token, pos + 1]));
    getNative().graphBegin();
    let graph = null;
    const temps = [];
    try {
      // with the guard on the captured step also clears the status words (the library moves the
      // checks' step number with the position at every replay)
      if (this.finitenessGuard) getNative().fillZero(this.tokenOut.ptr, 4, FINITENESS_STATUS_BYTES);
      await this.recordDecodeStep(createCommandRecorder('decode_capture'), temps, pos, { deviceKvLen: true });
    } finally {
      graph = getNative().graphEnd(pos);
    }
    getNative().graphSetMaxPosition(graph, c.maxSeq - 1);
    this.graph = graph;
    this.graphBuffers = temps;
    return first;
  }

  // One decode step by replaying the captured graph at position `pos`.
  async decodeStepGraph(token, pos) {
    const c = this.config;
    if (!(pos >= 0 && pos < c.maxSeq)) {
      throw new Error(`[decodeStepGraph] position ${pos} is outside the KV cache (maxSeq=${c.maxSeq})`);
    }
    if (!this.graph) return this.captureDecodeStep(token, pos);
    // token id and key count travel together; the attention kernels of the captured step read the count
    uploadData(this.ids, new Uint32Array([token, pos + 1]));
    getNative().graphLaunch(this.graph, pos);
    const bytes = await readBufferSlice(this.tokenOut, 0, this.finitenessGuard ? 4 + FINITENESS_STATUS_BYTES : 4);
    const words = new Uint32Array(bytes);
    if (this.finitenessGuard) {
      const status = parseFinitenessStatusWords(words, 1);
      if (status.triggered) throw new FinitenessError(`F16 bounds exceeded during generation${status.metadata}`);
    }
    return words[0];
  }

  releaseGraph() {
    if (this.graph) {
      getNative().graphDestroy(this.graph);
      for (const b of this.graphBuffers) releaseBuffer(b);
      this.graph = null;
      this.graphBuffers = [];
    }
  }

  destroy() {
    this.releaseGraph();
    this.releaseReadback();
    for (const l of this.layers) {
      for (const key of Object.keys(l)) releaseBuffer(l[key].buffer);
    }
  }
}
