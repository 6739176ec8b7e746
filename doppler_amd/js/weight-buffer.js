// Weight handle: reference src/gpu/weight-buffer.js:78-115,232-250.
// dtype is 'q4k' | 'f16' | 'f32'; Q4_K weights are always layout 'row' ([N, K] as
// N*ceil(K/256) raw 144-byte super-blocks, exactly what the RDRR loader uploads).

export function createWeightBuffer(buffer, dtype, layout, shape, label, materializations = null, metadata = null) {
  const mats = {};
  if (materializations && typeof materializations === 'object') {
    for (const key of Object.keys(materializations)) {
      const descriptor = materializations[key];
      if (descriptor && descriptor.buffer) {
        mats[key] = Object.freeze({ buffer: descriptor.buffer, layout: descriptor.layout || layout });
      }
    }
  }
  mats[dtype] = Object.freeze({ buffer, layout });
  const out = {
    buffer,
    dtype,
    layout,
    shape: Object.freeze([...shape]),
    label,
    materializations: Object.freeze(mats),
  };
  if (metadata) {
    out.metadata = metadata;
  }
  return out;
}

export function isWeightBuffer(value) {
  return !!value && typeof value === 'object' && 'buffer' in value && 'dtype' in value && 'layout' in value;
}

function isTensorLike(value) {
  return !!value && typeof value === 'object' && 'buffer' in value && 'dtype' in value && 'shape' in value;
}

export function getBuffer(weight) {
  if (isWeightBuffer(weight) || isTensorLike(weight)) return weight.buffer;
  return weight;
}

export function getLayout(weight) {
  return isWeightBuffer(weight) ? weight.layout : null;
}

export function getWeightDtype(weight) {
  if (isWeightBuffer(weight) || isTensorLike(weight)) return weight.dtype;
  return null;
}
