// Replays kernel plans on the GPU through HipBackend and reports the raw outputs.
//
//   node run_plan.js cases.json results.json
//
// cases.json: [{name, plan, inputs: [base64...]}]; results.json: [{name, output: base64}] (routine plans:
// [{name, outputs: [base64...]}]) plus the outcome of
// the Backend-protocol checks below (slot errors, refcounts, zero-size buffers, ranged reads), which restate
// src/backend.test.ts:88-135 for this device.
'use strict';

const fs = require('fs');
const { HipBackend, SlotError } = require('./hip_backend.js');

function check(cond, what) {
  if (!cond) throw new Error('check failed: ' + what);
}

function protocolChecks(be) {
  const a = be.malloc(12, new Uint8Array(new Float32Array([1, 2, 3]).buffer));
  check(Buffer.from(be.readSync(a)).equals(Buffer.from(new Float32Array([1, 2, 3]).buffer)), 'round trip');
  check(Buffer.from(be.readSync(a, 4, 4)).readFloatLE(0) === 2, 'ranged read');
  be.incRef(a);
  be.decRef(a);
  check(be.readSync(a).byteLength === 12, 'still alive after one of two decRefs');
  be.decRef(a);
  let threw = false;
  try { be.readSync(a); } catch (e) { threw = e instanceof SlotError; }
  check(threw, 'freed slot raises SlotError');
  threw = false;
  try { be.decRef(a); } catch (e) { threw = e instanceof SlotError; }
  check(threw, 'double free raises SlotError');
  const z = be.malloc(0);
  check(be.readSync(z).byteLength === 0, 'zero-size buffer');
  be.decRef(z);
  threw = false;
  try { be.malloc(8, new Uint8Array(4)); } catch (e) { threw = true; }
  check(threw, 'initialData size mismatch raises');
  return true;
}

// `read` must not block the thread: with a long queue of launches ahead of it the promise is still pending when the
// call returns, the event loop turns (setImmediate callbacks run) while the device works, and the bytes that arrive
// are those of a blocking read of the same slot.
function asyncReadCheck(be, c) {
  const ins = c.inputs.map((b64) => { const buf = Buffer.from(b64, 'base64'); return be.malloc(buf.length, buf); });
  const exe = be.prepareKernelSync(c.plan);
  const out = be.malloc(c.plan.outputBytes);
  be.dispatch(exe, ins, [out]);
  const want = Buffer.from(be.readSync(out));
  for (let i = 0; i < 400; ++i) be.dispatch(exe, ins, [out]);  // tens of milliseconds of queued device work
  let turns = 0, settled = false;
  const tick = () => { if (!settled) { turns++; setImmediate(tick); } };
  const p = be.read(out).then((bytes) => { settled = true; return Buffer.from(bytes); });
  const pendingAtReturn = !settled;
  setImmediate(tick);
  const empty = be.malloc(0);
  return p.then((got) => be.read(empty).then((none) => be.read(out, 4, 8).then((part) => {
    let threw = false;
    return be.read(987654).catch((e) => { threw = e instanceof SlotError; }).then(() => {
      ins.concat([out, empty]).forEach((s) => be.decRef(s));
      return { pendingAtReturn: pendingAtReturn, loopTurnsWhilePending: turns, bytesEqual: got.equals(want),
               emptyLength: none.byteLength, rangedEqual: Buffer.from(part).equals(want.slice(4, 12)), unknownSlotRejects: threw };
    });
  })));
}

function main() {
  const cases = JSON.parse(fs.readFileSync(process.argv[2], 'utf8'));
  const be = new HipBackend(0);
  const results = { device: be.info, protocol: protocolChecks(be), cases: [] };
  const asyncCase = cases.find((c) => c.asyncOnly === true);
  cases.forEach((c) => {
    if (c.asyncOnly === true) return;  // only for asyncReadCheck: its output is too large to report
    const ins = c.inputs.map((b64) => { const buf = Buffer.from(b64, 'base64'); return be.malloc(buf.length, buf); });
    if (c.plan.routine !== undefined) {
      const exe = be.prepareRoutineSync(c.plan);
      const outs = c.plan.outputBytes.map((b) => be.malloc(b));
      be.dispatch(exe, ins, outs);
      be.dispatch(exe, ins, outs);
      const raws = outs.map((o) => Buffer.from(be.readSync(o)).toString('base64'));
      ins.concat(outs).forEach((s) => be.decRef(s));
      results.cases.push({ name: c.name, outputs: raws });
      return;
    }
    const exe = be.prepareKernelSync(c.plan);
    const out = be.malloc(c.plan.outputBytes);
    be.dispatch(exe, ins, [out]);
    be.dispatch(exe, ins, [out]);  // a second dispatch of the same executable must give the same bytes
    const raw = Buffer.from(be.readSync(out));
    ins.concat([out]).forEach((s) => be.decRef(s));
    results.cases.push({ name: c.name, output: raw.toString('base64') });
  });
  const finish = () => {
    fs.writeFileSync(process.argv[3], JSON.stringify(results));
    console.log('ok ' + results.cases.length + ' cases on ' + be.info.name);
  };
  if (asyncCase === undefined) return finish();
  asyncReadCheck(be, asyncCase).then((r) => { results.asyncRead = r; finish(); }).catch((e) => { console.error(e); process.exit(1); });
}

main();
