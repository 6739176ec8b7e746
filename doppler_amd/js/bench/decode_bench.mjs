// Decode throughput of the JavaScript host: RDRR artifact -> JS loader -> HIP buffers -> prefill
// path -> timed decode loops through the op API (N-API addon -> C ABI): one blocking 4-byte token readback
// per step, then the generation loop with staged readback, then (graph) the captured step.  Prints one JSON line.
//   node doppler_amd/js/bench/decode_bench.mjs <artifact-dir> <prefill> <warmup> <steps> [graph]
import { initDevice } from '../kernel-selector.js';
import { HipTextDecoder } from '../pipeline/decode-step.js';
import { loadDecoderWeights } from '../loader/rdrr-loader.js';

const [dir, prefillArg, warmupArg, stepsArg, mode] = process.argv.slice(2);
const prefill = Number(prefillArg), warmup = Number(warmupArg), steps = Number(stepsArg);

async function timed(dec, step, tok, pos) {
  const t0 = process.hrtime.bigint();
  const tokens = [];
  for (let i = 0; i < steps; i++) {
    tok = await step(tok, pos + i);
    tokens.push(tok);
  }
  const seconds = Number(process.hrtime.bigint() - t0) / 1e9;
  return { tokens, tok, seconds };
}

async function main() {
  initDevice(0);
  const t0 = Date.now();
  const { config, weights } = loadDecoderWeights(dir, prefill + 2 * (warmup + steps) + 8);
  const dec = new HipTextDecoder(config, weights);
  const loadMs = Date.now() - t0;
  // seeded prompt ids (a linear congruential stream: the loader and the decode loop are what is measured)
  let s = 40;
  const prompt = Array.from({ length: prefill }, () => { s = (s * 1103515245 + 12345) % 2147483648; return s % config.vocab; });
  let tok = await dec.prefill(prompt, 0, { chunk: 2048 });
  let pos = prefill;
  for (let i = 0; i < warmup; i++) tok = await dec.decodeStep(tok, pos++);
  const eager = await timed(dec, (t, p) => dec.decodeStep(t, p), tok, pos);
  // the same positions again through the generation loop with staged readback (step k + 1 is enqueued from
  // the device-side token before the host waits for token k): the tokens must be the same
  await dec.decodeGreedy(tok, pos, Math.min(4, steps));
  const g0 = process.hrtime.bigint();
  const greedy = await dec.decodeGreedy(tok, pos, steps);
  const greedySeconds = Number(process.hrtime.bigint() - g0) / 1e9;
  pos += steps;
  const out = {
    host: 'javascript (node ' + process.version + ') -> N-API addon -> C ABI',
    tokens_per_s: steps / eager.seconds, ms_per_step: eager.seconds / steps * 1e3, load_ms: loadMs,
    tokens_head: eager.tokens.slice(0, 4),
    greedy_tokens_per_s: steps / greedySeconds, greedy_ms_per_step: greedySeconds / steps * 1e3,
    greedy_matches_blocking_steps: JSON.stringify(greedy) === JSON.stringify(eager.tokens),
  };
  if (mode === 'graph') {
    tok = await dec.captureDecodeStep(eager.tok, pos++);
    for (let i = 0; i < warmup; i++) tok = await dec.decodeStepGraph(tok, pos++);
    const g = await timed(dec, (t, p) => dec.decodeStepGraph(t, p), tok, pos);
    out.graph_tokens_per_s = steps / g.seconds;
    out.graph_ms_per_step = g.seconds / steps * 1e3;
    dec.releaseGraph();
  }
  console.log(JSON.stringify(out));
}
main().catch((e) => { console.error(e); process.exit(1); });
