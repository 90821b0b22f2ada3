// HipBackend: the reference's `Backend` interface (src/backend.ts:158-211) over the jaxhip N-API addon.
//
// Member for member what `src/backend/hip.ts` would hold in the reference tree: slots are opaque integers
// naming untyped device buffers with caller-managed reference counts; `dispatch` never blocks; reads are
// ordered after earlier dispatches because everything runs on one in-order stream.  Plain CommonJS without
// newer syntax, so it also loads on the Node 12 that ships with this image.
//
// Code generation is the one part not written in JavaScript here: `prepareKernelSync` takes a *plan* -- the
// HIP source texts and launch steps that the tuner and code generator produce for one Kernel (sources[],
// steps[{name, module, grid, block, shared, args}], scratchBytes[], compileOptions[], outputBytes) -- instead
// of the Kernel itself.  In the reference tree the plan is computed in-process by the TypeScript port of
// tuneHip/kernelgen; everything below that point is identical.
'use strict';

const path = require('path');
const addon = require(path.join(__dirname, 'jaxhip.node'));

class SlotError extends Error {  // src/backend.ts:222-226
  constructor(slot) {
    super('Used a buffer that is invalid or already freed: ' + slot);
    this.name = 'SlotError';
  }
}

class Executable {  // src/backend.ts:213-220
  constructor(source, data) {
    this.source = source;
    this.data = data;
  }
}

const ROUND = 256n;

class HipBackend {
  constructor(device) {
    this.type = 'hip';
    this.maxArgs = 64;
    addon.init(device === undefined ? 0 : device);
    this.info = addon.deviceInfo();
    this._slots = new Map();  // slot -> {ptr: BigInt, size: number, ref: number}
    this._next = 1;
    this._pool = new Map();   // rounded size -> [ptr]; safe to recycle at once: one in-order stream
    this._exes = new Map();   // plan key -> Executable
  }

  // -- memory ------------------------------------------------------------------------------------------
  _rounded(size) {
    const s = BigInt(size);
    return s === 0n ? ROUND : ((s + ROUND - 1n) / ROUND) * ROUND;
  }

  malloc(size, initialData) {
    if (initialData !== undefined && initialData.byteLength !== size) {
      throw new Error('initialData size does not match buffer size');  // src/backend/cpu.ts:22-24
    }
    const cls = this._rounded(size);
    const free = this._pool.get(cls);
    const ptr = free !== undefined && free.length ? free.pop() : addon.malloc(cls);
    if (initialData !== undefined && size > 0) {
      addon.h2d(ptr, new Uint8Array(initialData.buffer, initialData.byteOffset, initialData.byteLength));
    }
    const slot = this._next++;
    this._slots.set(slot, { ptr: ptr, size: size, ref: 1 });
    return slot;
  }

  _get(slot) {
    const s = this._slots.get(slot);
    if (s === undefined) throw new SlotError(slot);
    return s;
  }

  incRef(slot) {
    this._get(slot).ref++;
  }

  decRef(slot) {
    const s = this._get(slot);
    if (--s.ref === 0) {
      this._slots.delete(slot);
      const cls = this._rounded(s.size);
      if (!this._pool.has(cls)) this._pool.set(cls, []);
      this._pool.get(cls).push(s.ptr);
    }
  }

  readSync(slot, start, count) {
    const s = this._get(slot);
    start = start === undefined ? 0 : start;
    count = count === undefined ? s.size - start : count;
    if (start < 0 || count < 0 || start + count > s.size) throw new RangeError('read outside of the buffer');
    return addon.d2h(s.ptr, start, count);
  }

  // Asynchronous read (src/backend.ts:182-186; src/backend/webgpu/reader.ts maps a staging buffer the same way): the
  // copy into pinned host memory is queued behind every earlier dispatch, and the promise resolves from the event
  // loop once the copy's completion event has passed -- the thread is never blocked on the device, so a caller that
  // awaits a result goes on preparing and dispatching other work.
  read(slot, start, count) {
    return new Promise((resolve, reject) => {
      let pending;
      try {
        const s = this._get(slot);
        start = start === undefined ? 0 : start;
        count = count === undefined ? s.size - start : count;
        if (start < 0 || count < 0 || start + count > s.size) throw new RangeError('read outside of the buffer');
        pending = addon.d2hAsync(s.ptr, start, count);
      } catch (e) {
        reject(e);
        return;
      }
      const poll = () => {
        try {
          if (!addon.eventQuery(pending.event)) {
            setImmediate(poll);
            return;
          }
          addon.eventDestroy(pending.event);
          pending.event = undefined;
          resolve(pending.data);
        } catch (e) {
          if (pending.event !== undefined) {
            try { addon.eventDestroy(pending.event); } catch (_) { /* the first error is the one to report */ }
            pending.event = undefined;
          }
          reject(e);
        }
      };
      poll();
    });
  }

  // -- kernels -----------------------------------------------------------------------------------------
  prepareKernelSync(plan) {
    const key = plan.key;
    if (key !== undefined && this._exes.has(key)) return this._exes.get(key);
    const modules = plan.sources.map((src, i) => addon.moduleLoad(addon.compile(src, 'plan' + i + '.hip', plan.compileOptions)));
    const functions = plan.steps.map((st) => addon.moduleFunction(modules[st.module], st.name));
    const scratch = plan.scratchBytes.map((b) => addon.malloc(this._rounded(b)));
    const exe = new Executable(plan, { modules: modules, functions: functions, scratch: scratch });
    if (key !== undefined) this._exes.set(key, exe);
    return exe;
  }

  prepareKernel(plan) {
    return Promise.resolve().then(() => this.prepareKernelSync(plan));
  }

  // A routine plan (`routine`, `inputBytes[]`, `outputBytes[]` beside the common fields) prepares exactly like a
  // kernel plan: compile, load, look the entry points up, allocate scratch (src/backend.ts:197-203).
  prepareRoutineSync(plan) {
    if (plan.routine === undefined) throw new Error('prepareRoutineSync expects a routine plan');
    return this.prepareKernelSync(plan);
  }

  prepareRoutine(plan) {
    return Promise.resolve().then(() => this.prepareRoutineSync(plan));
  }

  _dispatchRoutine(exe, ins, outs) {
    const plan = exe.source;
    if (ins.length !== plan.inputBytes.length || outs.length !== plan.outputBytes.length) {
      throw new Error(plan.routine + ' takes ' + plan.inputBytes.length + ' inputs and ' + plan.outputBytes.length + ' outputs');
    }
    plan.inputBytes.forEach((b, i) => {
      if (ins[i].size < b) throw new Error('input ' + i + ' holds ' + ins[i].size + ' bytes, the routine addresses ' + b);
    });
    plan.outputBytes.forEach((b, i) => {
      if (outs[i].size < b) throw new Error('output ' + i + ' holds ' + outs[i].size + ' bytes, the routine addresses ' + b);
    });
    plan.steps.forEach((st, i) => {
      const args = st.args.map((a) => {
        if (a[0] === 'in') return ins[a[1]].ptr;
        if (a[0] === 'out') return outs[a[1]].ptr;
        if (a[0] === 'scratch') return exe.data.scratch[a[1]];
        return BigInt(a[1]);  // by-value 64-bit integer: same 8-byte argument cell as a pointer
      });
      addon.launch(exe.data.functions[i], st.grid, st.block, st.shared, args);
    });
  }

  dispatch(exe, inputs, outputs) {
    const plan = exe.source;
    const ins = inputs.map((s) => this._get(s));
    const outs = outputs.map((s) => this._get(s));
    if (plan.routine !== undefined) return this._dispatchRoutine(exe, ins, outs);
    if (outs.length !== 1) throw new Error('a Kernel has exactly one output');
    if (outs[0].size < plan.outputBytes) {
      throw new Error('output slot holds ' + outs[0].size + ' bytes, kernel writes ' + plan.outputBytes);
    }
    const need = plan.minInputBytes || {};
    Object.keys(need).forEach((gid) => {
      if (ins[gid] === undefined || ins[gid].size < need[gid]) {
        throw new Error('input ' + gid + ' is smaller than the ' + need[gid] + ' bytes the kernel addresses');
      }
    });
    if (plan.size === 0) return;
    plan.steps.forEach((st, i) => {
      const ptrs = st.args.map((a) => {
        if (a[0] === 'in') return ins[a[1]].ptr;
        if (a[0] === 'out') return outs[0].ptr;
        return exe.data.scratch[a[1]];
      });
      addon.launch(exe.data.functions[i], st.grid, st.block, st.shared, ptrs);
    });
  }

  sync() {
    addon.sync();
  }
}

module.exports = { HipBackend: HipBackend, SlotError: SlotError, Executable: Executable, addon: addon };
