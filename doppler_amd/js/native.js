// Loads the Node-API addon (doppler_hip.node, built by `python -m doppler_amd.build`).
// There is no other backend: if the addon is missing every op fails at import time.
import { createRequire } from 'module';
import { fileURLToPath } from 'url';
import { dirname, join } from 'path';

const here = dirname(fileURLToPath(import.meta.url));
const require = createRequire(import.meta.url);

let native;
try {
  native = require(join(here, 'doppler_hip.node'));
} catch (error) {
  throw new Error(
    `[doppler-hip] native addon not available (${error.message}). ` +
    'Build it with `python -m doppler_amd.build`; the HIP path has no fallback.'
  );
}

export const DTYPE = Object.freeze({ f32: 0, f16: 1 });
export const ACT = Object.freeze({ silu: 0, gelu: 1 });
export const KV_LAYOUT = Object.freeze({ contiguous: 0, ring: 1 });

let initialised = false;

// Reference: initDevice() (src/gpu/device.js:605-700).  One device, one queue.
export function initDevice(ordinal = 0) {
  if (!initialised) {
    native.init(ordinal);
    initialised = true;
  }
  return native;
}

export function getNative() {
  if (!initialised) {
    initDevice(0);
  }
  return native;
}

export default native;
