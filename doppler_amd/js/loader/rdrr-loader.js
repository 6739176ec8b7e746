// RDRR artifact (manifest.json + shard_NNNNN.bin) -> weights of the HIP text decoder.
//
// The part of the reference's loader this path needs:
//   manifest normalisation   src/formats/rdrr/parsing.js:28-76 (filename | fileName, running
//                            shard offsets), tensor locations :78-160 (shard | shardIndex,
//                            offset, size, shape, spans across shards; same error texts)
//   Q4_K_M tensors           uploaded byte for byte, layout 'row'
//                            (src/loader/tensors/tensor-loader.js:540-555)
//   f16 norm weights         widened to f32 on the host (tensor-loader.js:520-533)
//   RoPE tables              frequency rounded to f32, angle and cos/sin in f64, stored f32
//                            (src/inference/pipelines/text/init-rope.js:21-26,120-133)
// Unsupported model features fail closed with the field named in the message.  A shard that
// carries a sha256 hash is checked against it when first opened.
import crypto from 'crypto';
import fs from 'fs';
import path from 'path';

const QK = 256, BLOCK_BYTES = 144;
const DTYPE_BYTES = { F32: 4, F16: 2, BF16: 2 };

export function shardFilename(index) {
  return `shard_${String(index).padStart(5, '0')}.bin`;
}

function expectedBytes(name, loc) {
  if (loc.dtype === 'Q4_K_M') {
    if (loc.shape.length !== 2) throw new Error(`Tensor '${name}' is Q4_K_M but not 2-D`);
    return loc.shape[0] * Math.ceil(loc.shape[1] / QK) * BLOCK_BYTES;
  }
  if (DTYPE_BYTES[loc.dtype]) return loc.shape.reduce((a, b) => a * b, 1) * DTYPE_BYTES[loc.dtype];
  return null;
}

export function parseManifest(jsonString) {
  let manifest;
  try {
    manifest = JSON.parse(jsonString);
  } catch (e) {
    throw new Error(`Failed to parse manifest JSON: ${e.message}`);
  }
  const errors = [];
  if (!Array.isArray(manifest.shards) || manifest.shards.length === 0) errors.push('Missing or empty shards array');
  let offset = 0;
  manifest.shards = (manifest.shards || []).map((shard, i) => {
    const normalized = {
      index: shard.index !== undefined ? shard.index : i,
      filename: shard.filename || shard.fileName || '',
      size: shard.size,
      hash: shard.hash || shard.blake3 || '',
      offset: shard.offset !== undefined ? shard.offset : offset,
    };
    if (typeof shard.size !== 'number' || shard.size <= 0) errors.push(`Shard ${i} has invalid size`);
    if (normalized.filename && (path.basename(normalized.filename) !== normalized.filename || normalized.filename === '.' || normalized.filename === '..')) {
      errors.push(`Shard ${i} filename '${normalized.filename}' must be a plain file name inside the artifact directory`);
    }
    offset += shard.size;
    return normalized;
  });
  const hasTensors = manifest.tensors && typeof manifest.tensors === 'object';
  if (!hasTensors && typeof manifest.tensorsFile !== 'string') errors.push('Missing tensorsFile and tensors - one is required');
  if (errors.length) throw new Error(`Invalid manifest:\n  - ${errors.join('\n  - ')}`);
  if (hasTensors) manifest.tensors = parseTensorMap(manifest.tensors, manifest.shards);
  return manifest;
}

export function parseTensorMap(tensorMap, shards) {
  const out = {};
  for (const [name, loc] of Object.entries(tensorMap)) {
    if (!Array.isArray(loc.shape)) throw new Error(`Tensor '${name}' missing shape`);
    let spans;
    if (loc.spans !== undefined) {
      if (!Array.isArray(loc.spans)) throw new Error(`Tensor '${name}' has invalid spans array`);
      spans = loc.spans.map((span, j) => {
        const idx = span && typeof span.shardIndex === 'number' ? span.shardIndex : span && span.shard;
        if (typeof idx !== 'number') throw new Error(`Tensor '${name}' span[${j}] missing shard index`);
        if (typeof span.offset !== 'number') throw new Error(`Tensor '${name}' span[${j}] missing offset`);
        if (typeof span.size !== 'number') throw new Error(`Tensor '${name}' span[${j}] missing size`);
        return { shardIndex: idx, offset: span.offset, size: span.size };
      });
    } else {
      const idx = typeof loc.shardIndex === 'number' ? loc.shardIndex : loc.shard;
      if (typeof idx !== 'number') throw new Error(`Tensor '${name}' missing shard index`);
      if (typeof loc.offset !== 'number') throw new Error(`Tensor '${name}' missing offset`);
      if (typeof loc.size !== 'number') throw new Error(`Tensor '${name}' missing size`);
      spans = [{ shardIndex: idx, offset: loc.offset, size: loc.size }];
    }
    const covered = spans.reduce((a, s) => a + s.size, 0);
    const size = typeof loc.size === 'number' ? loc.size : covered;
    if (covered !== size) throw new Error(`Tensor '${name}' spans cover ${covered} bytes, size says ${size}`);
    for (const s of spans) {
      if (s.shardIndex < 0 || s.shardIndex >= shards.length) throw new Error(`Tensor '${name}' names shard ${s.shardIndex} of ${shards.length}`);
      if (s.offset < 0 || s.offset + s.size > shards[s.shardIndex].size) throw new Error(`Tensor '${name}' reaches past the end of shard ${s.shardIndex}`);
    }
    const want = expectedBytes(name, loc);
    if (want !== null && want !== size) {
      throw new Error(`Tensor '${name}' (${loc.dtype} [${loc.shape}]) should hold ${want} bytes, manifest says ${size}`);
    }
    out[name] = Object.assign({}, loc, { size, spans });
  }
  return out;
}

function unsupported(what) {
  throw new Error(`[rdrr] unsupported by the HIP decode path: ${what}`);
}

export function decoderConfig(manifest, maxSeq) {
  const a = manifest.architecture || {}, inf = manifest.inference || {};
  for (const k of ['numLayers', 'hiddenSize', 'intermediateSize', 'numAttentionHeads', 'numKeyValueHeads', 'headDim', 'vocabSize']) {
    if (typeof a[k] !== 'number') throw new Error(`Invalid manifest:\n  - architecture.${k} is missing`);
  }
  const att = inf.attention || {}, nrm = inf.normalization || {}, ffn = inf.ffn || {}, rope = inf.rope || {}, out = inf.output || {};
  if (manifest.moeConfig) unsupported('moeConfig (mixture of experts)');
  if (((manifest.quantizationInfo || {}).layout || 'row') !== 'row') unsupported("quantizationInfo.layout != 'row'");
  if (att.slidingWindow) unsupported('inference.attention.slidingWindow');
  if (att.attnLogitSoftcapping) unsupported('inference.attention.attnLogitSoftcapping');
  if (att.attentionBias || att.attentionOutputGate || att.valueNorm) unsupported('attention bias / output gate / value norm');
  if (nrm.preFeedforwardNorm || nrm.postFeedforwardNorm) unsupported('pre/post feed-forward norms');
  if (nrm.rmsNormWeightOffset) unsupported('rmsNormWeightOffset in the decoder host');
  if (ffn.gatedActivation === false || (ffn.branchMode || 'dense') !== 'dense') unsupported('non-gated or non-dense FFN');
  if ((ffn.activation || 'silu') !== 'silu' || ffn.swigluLimit) unsupported(`ffn.activation ${ffn.activation} / swigluLimit in the decoder host`);
  if (rope.partialRotaryFactor || rope.ropeScalingType || rope.mropeSection) unsupported('partial / scaled / multi-axis RoPE');
  if (out.tieWordEmbeddings === false) unsupported('untied LM head');
  if (out.finalLogitSoftcapping || out.scaleEmbeddings) unsupported('logit soft cap / embedding scale');
  if (((inf.layerPattern || {}).type || 'uniform') !== 'uniform') unsupported('non-uniform layer pattern');
  // scalars the decoder hard-wires: attention scale 1/sqrt(headDim), no logit or residual-branch scale
  if (att.queryPreAttnScalar !== undefined && att.queryPreAttnScalar !== null && att.queryPreAttnScalar !== a.headDim) {
    unsupported(`inference.attention.queryPreAttnScalar ${att.queryPreAttnScalar} != headDim ${a.headDim}`);
  }
  if (out.logitInputScale !== undefined && out.logitInputScale !== null && out.logitInputScale !== 1) {
    unsupported(`inference.output.logitInputScale ${out.logitInputScale}`);
  }
  const rbs = (inf.layerPattern || {}).residualBranchScale;
  if (rbs !== undefined && rbs !== null && rbs !== 1) unsupported(`inference.layerPattern.residualBranchScale ${rbs}`);
  return {
    layers: a.numLayers, hidden: a.hiddenSize, inter: a.intermediateSize, heads: a.numAttentionHeads,
    kvHeads: a.numKeyValueHeads, headDim: a.headDim, vocab: a.vocabSize,
    eps: typeof nrm.rmsNormEps === 'number' ? nrm.rmsNormEps : 1e-6, qkNorm: !!att.queryKeyNorm,
    theta: rope.ropeTheta || a.ropeTheta || 10000, maxSeq,
  };
}

export function ropeTables(rotaryDim, maxSeq, theta) {
  const half = rotaryDim / 2;
  const cos = new Float32Array(maxSeq * half), sin = new Float32Array(maxSeq * half);
  for (let i = 0; i < half; i++) {
    const freq = Math.fround(1 / Math.pow(theta, (2 * i) / rotaryDim));
    for (let p = 0; p < maxSeq; p++) {
      cos[p * half + i] = Math.cos(p * freq);
      sin[p * half + i] = Math.sin(p * freq);
    }
  }
  return { cos, sin };
}

function halfToFloat(bits) {
  const sign = (bits & 0x8000) ? -1 : 1, exp = (bits >> 10) & 0x1f, frac = bits & 0x3ff;
  if (exp === 0) return sign * frac * Math.pow(2, -24);
  if (exp === 31) return frac ? NaN : sign * Infinity;
  return sign * (1 + frac / 1024) * Math.pow(2, exp - 15);
}

export class RdrrArtifact {
  // verifyHashes: check each shard that carries a hash against it when first opened (sha256 only;
  // a hashed shard under another algorithm is refused unless this is off).
  constructor(dir, { verifyHashes = true } = {}) {
    this.dir = dir;
    this.verifyHashes = verifyHashes;
    this.manifest = parseManifest(fs.readFileSync(path.join(dir, 'manifest.json'), 'utf8'));
    if (!this.manifest.tensors || typeof this.manifest.tensors !== 'object') {
      let raw;
      try {
        raw = JSON.parse(fs.readFileSync(path.join(dir, this.manifest.tensorsFile), 'utf8'));
      } catch (e) {
        throw new Error(`Failed to parse tensors.json: ${e.message}`);
      }
      this.manifest.tensors = parseTensorMap(raw, this.manifest.shards);
    }
    this.tensors = this.manifest.tensors;
    this.fds = new Map();
  }

  shardFd(index) {
    if (!this.fds.has(index)) {
      const info = this.manifest.shards[index];
      const p = path.join(this.dir, info.filename || shardFilename(index));
      if (!fs.existsSync(p)) throw new Error(`Shard file ${p} is missing`);
      const onDisk = fs.statSync(p).size;
      if (onDisk !== info.size) throw new Error(`Shard ${index} is ${onDisk} bytes on disk, manifest says ${info.size}`);
      const fd = fs.openSync(p, 'r');
      if (this.verifyHashes && info.hash) {
        const algorithm = this.manifest.hashAlgorithm;
        if (algorithm !== 'sha256') {
          fs.closeSync(fd);
          throw new Error(`Shard ${index} carries a ${algorithm} hash, which this loader cannot check (pass verifyHashes: false to load it unchecked)`);
        }
        const h = crypto.createHash('sha256'), buf = Buffer.allocUnsafe(16 << 20);
        for (let at = 0; at < info.size;) {
          const n = fs.readSync(fd, buf, 0, Math.min(buf.length, info.size - at), at);
          if (n <= 0) break;
          h.update(buf.subarray(0, n));
          at += n;
        }
        const got = h.digest('hex');
        if (got !== String(info.hash).toLowerCase()) {
          fs.closeSync(fd);
          throw new Error(`Shard ${index} fails its sha256 check (manifest ${info.hash}, file ${got})`);
        }
      }
      this.fds.set(index, fd);
    }
    return this.fds.get(index);
  }

  find(...candidates) {
    for (const c of candidates) for (const prefix of ['', 'model.']) if (this.tensors[prefix + c]) return prefix + c;
    throw new Error(`Tensor '${candidates[0]}' is not in the manifest`);
  }

  tensorBytes(name) {
    const loc = this.tensors[name];
    if (!loc) throw new Error(`Tensor '${name}' is not in the manifest`);
    const out = new Uint8Array(loc.size);
    let at = 0;
    for (const s of loc.spans) {
      let done = 0;
      while (done < s.size) {
        const n = fs.readSync(this.shardFd(s.shardIndex), out, at + done, s.size - done, s.offset + done);
        if (n <= 0) throw new Error(`Tensor '${name}': short read from shard ${s.shardIndex}`);
        done += n;
      }
      at += s.size;
    }
    return out;
  }

  tensorF32(name) {
    const loc = this.tensors[name], raw = this.tensorBytes(name);
    if (loc.dtype === 'F32') return new Float32Array(raw.buffer, raw.byteOffset, raw.byteLength / 4);
    if (loc.dtype !== 'F16') throw new Error(`Tensor '${name}' has dtype ${loc.dtype} where f16/f32 is expected`);
    const h = new Uint16Array(raw.buffer, raw.byteOffset, raw.byteLength / 2), f = new Float32Array(h.length);
    for (let i = 0; i < h.length; i++) f[i] = halfToFloat(h[i]);
    return f;
  }

  close() {
    for (const fd of this.fds.values()) fs.closeSync(fd);
    this.fds.clear();
  }
}

function concat(parts) {
  const out = new Uint8Array(parts.reduce((a, p) => a + p.byteLength, 0));
  let at = 0;
  for (const p of parts) { out.set(p, at); at += p.byteLength; }
  return out;
}

// {config, weights} in the form HipTextDecoder takes (pipeline/decode-step.js).
export function loadDecoderWeights(dir, maxSeq) {
  const art = new RdrrArtifact(dir);
  try {
    const c = decoderConfig(art.manifest, maxSeq);
    const q4 = (name, shape) => {
      const loc = art.tensors[name];
      if (loc.dtype !== 'Q4_K_M' || (loc.layout || 'row') !== 'row') {
        throw new Error(`Tensor '${name}' must be Q4_K_M in row layout (dtype ${loc.dtype}, layout ${loc.layout})`);
      }
      if (loc.shape[0] !== shape[0] || loc.shape[1] !== shape[1]) {
        throw new Error(`Tensor '${name}' has shape [${loc.shape}], architecture implies [${shape}]`);
      }
      return art.tensorBytes(name);
    };
    const qs = c.heads * c.headDim, ks = c.kvHeads * c.headDim;
    const ones = () => new Float32Array(c.headDim).fill(1);
    const layers = [];
    for (let i = 0; i < c.layers; i++) {
      const t = (s) => art.find(`layers.${i}.${s}`);
      layers.push({
        wqkv: concat([q4(t('self_attn.q_proj.weight'), [qs, c.hidden]), q4(t('self_attn.k_proj.weight'), [ks, c.hidden]),
          q4(t('self_attn.v_proj.weight'), [ks, c.hidden])]),
        wo: q4(t('self_attn.o_proj.weight'), [c.hidden, qs]),
        wgate: q4(t('mlp.gate_proj.weight'), [c.inter, c.hidden]),
        wup: q4(t('mlp.up_proj.weight'), [c.inter, c.hidden]),
        wdown: q4(t('mlp.down_proj.weight'), [c.hidden, c.inter]),
        inputNorm: art.tensorF32(t('input_layernorm.weight')),
        postAttnNorm: art.tensorF32(t('post_attention_layernorm.weight')),
        qNorm: c.qkNorm ? art.tensorF32(t('self_attn.q_norm.weight')) : ones(),
        kNorm: c.qkNorm ? art.tensorF32(t('self_attn.k_norm.weight')) : ones(),
      });
    }
    const ename = art.find('embed_tokens.weight'), eloc = art.tensors[ename];
    if (eloc.dtype !== 'F16' || eloc.shape[0] !== c.vocab || eloc.shape[1] !== c.hidden) {
      throw new Error(`Tensor '${ename}' must be F16 [${c.vocab}, ${c.hidden}] (dtype ${eloc.dtype}, shape [${eloc.shape}])`);
    }
    const { cos, sin } = ropeTables(c.headDim, maxSeq, c.theta);
    return {
      config: c,
      weights: { layers, embed: art.tensorBytes(ename), finalNorm: art.tensorF32(art.find('norm.weight')), cos, sin },
    };
  } finally {
    art.close();
  }
}
