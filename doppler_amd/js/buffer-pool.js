// Device buffers for the HIP path.  Mirrors the calls the reference's ops and pipeline make
// on src/memory/buffer-pool.js:815-869: acquireBuffer / releaseBuffer / uploadData /
// readBuffer.  A buffer is { ptr (BigInt device address), size, label }.  Released buffers
// are kept in size buckets and handed out again; everything runs on one stream, so a buffer
// released after an op was enqueued cannot be overwritten before that op has run.
import { getNative } from './native.js';

const ALIGN = 256;
const free = new Map();      // bucket size -> HipBuffer[]
const active = new Set();

export class HipBuffer {
  constructor(ptr, size, capacity, label) {
    this.ptr = ptr;
    this.size = size;
    this.capacity = capacity;
    this.label = label || null;
  }

  destroy() {
    discardBuffer(this);
  }
}

function bucketOf(size) {
  const n = Math.max(ALIGN, Math.ceil(size / ALIGN) * ALIGN);
  // power-of-two buckets above 64 KiB keep the free lists short
  if (n <= 65536) return n;
  return Math.pow(2, Math.ceil(Math.log2(n)));
}

export function acquireBuffer(size, usage, label) {
  if (!Number.isFinite(size) || size <= 0) {
    throw new Error(`[BufferPool] invalid buffer size ${size}`);
  }
  const native = getNative();
  const cap = bucketOf(size);
  const list = free.get(cap);
  let buf;
  if (list && list.length > 0) {
    buf = list.pop();
    buf.size = size;
    buf.label = label || null;
  } else {
    const ptr = native.malloc(cap);
    native.fillZero(ptr, 0, cap);      // fresh WebGPU buffers read as zero; keep that
    buf = new HipBuffer(ptr, size, cap, label);
  }
  active.add(buf);
  return buf;
}

export function releaseBuffer(buffer) {
  if (!buffer || !active.has(buffer)) return;
  active.delete(buffer);
  let list = free.get(buffer.capacity);
  if (!list) {
    list = [];
    free.set(buffer.capacity, list);
  }
  list.push(buffer);
}

export function discardBuffer(buffer) {
  if (!buffer || buffer.ptr === null) return;
  active.delete(buffer);
  getNative().free(buffer.ptr);
  buffer.ptr = null;
}

export function isBufferActive(buffer) {
  return active.has(buffer);
}

export function uploadData(buffer, data, offset = 0) {
  const bytes = data.byteLength;
  if (offset + bytes > buffer.capacity) {
    throw new Error(`[BufferPool] upload of ${bytes} bytes at ${offset} exceeds buffer of ${buffer.capacity}`);
  }
  getNative().upload(buffer.ptr, offset, data);
}

// Waits for all queued work, like mapAsync on a staging copy in the reference.
export async function readBuffer(buffer, size) {
  const bytes = size === undefined || size === null ? buffer.size : size;
  return getNative().download(buffer.ptr, 0, bytes);
}

export async function readBufferSlice(buffer, offset, size) {
  return getNative().download(buffer.ptr, offset, size);
}

export function poolStats() {
  let pooled = 0;
  for (const list of free.values()) pooled += list.length;
  return { active: active.size, pooled };
}
