'use strict';
// Minimal test harness (node 12 has no test runner): it(name, fn) collects, run() reports.
const path = require('path');
const core = require(path.join(__dirname, '..', '..', 'mlx-node_amd', 'bin', 'mxopt.node'));

const cases = [];
function it(name, fn) { cases.push([name, fn]); }

// vitest's toBeCloseTo: |a - b| < 10^-digits / 2
function close(a, b, digits = 2) { return Math.abs(a - b) < Math.pow(10, -digits) / 2; }
function check(cond, what) { if (!cond) throw new Error('expected ' + what); }

function f32(values, dims) {
  const data = values instanceof Float32Array ? values : new Float32Array(values);
  return core.MxArray.fromFloat32(data, BigInt64Array.from((dims || [data.length]).map((d) => BigInt(d))));
}

function run() {
  let failed = 0;
  for (const [name, fn] of cases) {
    try {
      fn();
      console.log('PASS ' + name);
    } catch (e) {
      failed += 1;
      console.log('FAIL ' + name + ': ' + (e && e.stack ? e.stack.split('\n').slice(0, 3).join(' | ') : e));
    }
  }
  console.log(`${cases.length - failed} passed, ${failed} failed`);
  process.exit(failed ? 1 : 0);
}

module.exports = { core, it, close, check, f32, run };
