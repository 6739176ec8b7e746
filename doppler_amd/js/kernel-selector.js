// Entry module of the HIP path, the counterpart of the reference's src/gpu/kernel-selector.js:
// re-exports every op plus the handle, buffer and recorder helpers the pipeline uses.
export * from './kernels/index.js';
export { createTensor, dtypeBytes, tensorBytes } from './tensor.js';
export { createWeightBuffer, isWeightBuffer, getBuffer, getLayout, getWeightDtype } from './weight-buffer.js';
export { acquireBuffer, releaseBuffer, discardBuffer, uploadData, readBuffer, readBufferSlice, isBufferActive, poolStats } from './buffer-pool.js';
export { CommandRecorder, createCommandRecorder, createProfilingRecorder } from './command-recorder.js';
export { initDevice } from './native.js';
