// CommandRecorder for the HIP path (reference: src/gpu/command-recorder.js:14,353-560,723-728).
//
// The reference batches a decode step's dispatches into one command encoder and submits
// once.  HIP ops are enqueued on one stream as they are recorded, so recording IS
// submission: submit() only recycles the temporaries, submitAndWait() also drains the
// stream.  A profiling recorder (createProfilingRecorder) brackets every recorded op with
// HIP events on the op stream, the counterpart of the reference's timestamp-query
// profiling (command-recorder.js:116-140); resolveProfileTimings() returns milliseconds
// summed per label, as the reference's accessor of the same name does (:622-700).
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
    // profiling: events[i] is recorded after op i - 1 (events[0] when the recorder is created),
    // so op i ran between events[i] and events[i + 1] on the stream
    this.events = [];
    this.labels = [];
    if (this.profiling) this.events.push(this.recordEvent());
  }

  recordEvent() {
    const native = getNative();
    const ev = native.eventCreate();
    native.eventRecord(ev);
    return ev;
  }

  isProfilingEnabled() {
    return this.profiling;
  }

  beginComputePass() {
    return this;
  }

  noteDispatch(label) {
    this.opCount += 1;
    if (this.profiling) {
      this.labels.push(label);
      this.events.push(this.recordEvent());
    }
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

  // { label: milliseconds } summed over the ops recorded under each label; null when the
  // recorder does not profile.  Waits for the recorded work.
  async resolveProfileTimings() {
    if (!this.profiling) return null;
    if (!this.submitted) {
      throw new Error('[CommandRecorder] Must submit before resolving timings');
    }
    const native = getNative();
    const timings = {};
    for (let i = 0; i < this.labels.length; i++) {
      const ms = native.eventElapsedMs(this.events[i], this.events[i + 1]);
      if (ms < 0 || ms > 60000) continue;
      timings[this.labels[i]] = (timings[this.labels[i]] || 0) + ms;
    }
    for (const ev of this.events) native.eventDestroy(ev);
    this.events = [];
    this.labels = [];
    return timings;
  }

  static formatProfileReport(timings) {
    const entries = Object.entries(timings).sort((a, b) => b[1] - a[1]);
    const total = entries.reduce((sum, e) => sum + e[1], 0);
    const lines = ['GPU Profile Report', 'Kernel'.padEnd(36) + 'Time (ms)'.padStart(12) + '%'.padStart(8)];
    for (const [label, time] of entries) {
      lines.push(label.padEnd(36) + time.toFixed(3).padStart(12) + (time / total * 100).toFixed(1).padStart(8));
    }
    lines.push('TOTAL'.padEnd(36) + total.toFixed(3).padStart(12) + '100.0'.padStart(8));
    return lines.join('\n');
  }
}

export function createCommandRecorder(label) {
  return new CommandRecorder(label);
}

export function createProfilingRecorder(label) {
  return new CommandRecorder(label, { profile: true });
}
