'use strict';
/** Minimal test harness for the Node-side tests (no test framework is installed). */
const fs = require('fs');
const path = require('path');

const tests = [];

function test(name, fn) {
  tests.push({name, fn});
}

async function run(title) {
  let failed = 0;
  const filter = process.env.TEST_FILTER;
  for (const t of tests) {
    if (filter && t.name.indexOf(filter) === -1) {
      continue;
    }
    try {
      await t.fn();
      if (process.env.TEST_VERBOSE) {
        console.log(`ok   ${t.name}`);
      }
    } catch (e) {
      failed++;
      console.log(`FAIL ${t.name}\n     ${(e.stack || e.message).split('\n').slice(0, 6).join('\n     ')}`);
    }
  }
  console.log(`${title}: ${tests.length - failed} passed, ${failed} failed`);
  process.exitCode = failed ? 1 : 0;
}

function assert(cond, msg) {
  if (!cond) {
    throw new Error(msg || 'assertion failed');
  }
}

function assertEqual(a, b, msg) {
  if (JSON.stringify(a) !== JSON.stringify(b)) {
    throw new Error(`${msg || 'not equal'}: ${JSON.stringify(a)} vs ${JSON.stringify(b)}`);
  }
}

function assertThrows(fn, pattern) {
  let threw = null;
  try {
    fn();
  } catch (e) {
    threw = e;
  }
  if (!threw) {
    throw new Error(`expected an error matching ${pattern}`);
  }
  if (pattern && !pattern.test(threw.message)) {
    throw new Error(`error "${threw.message}" does not match ${pattern}`);
  }
}

/** expectArraysClose of tfjs-core/src/test_util.ts:63-111 (epsilon 1e-3 on float32 backends). */
function assertClose(actual, expected, eps) {
  eps = eps == null ? 1e-3 : eps;
  assert(actual.length === expected.length, `length ${actual.length} vs ${expected.length}`);
  for (let i = 0; i < expected.length; i++) {
    const a = actual[i], e = expected[i];
    if (Number.isNaN(a) && Number.isNaN(e)) {
      continue;
    }
    if (!(Math.abs(a - e) <= eps)) {
      throw new Error(`element ${i}: got ${a}, want ${e}`);
    }
  }
}

/** The build's acceptance bound: max |d| <= tol * max(1, |ref|). */
function assertParity(actual, expected, tol) {
  tol = tol == null ? 1e-3 : tol;
  assert(actual.length === expected.length, `length ${actual.length} vs ${expected.length}`);
  for (let i = 0; i < expected.length; i++) {
    const a = actual[i], e = expected[i];
    if (Number.isNaN(a) && Number.isNaN(e)) {
      continue;
    }
    if (!(Math.abs(a - e) <= tol * Math.max(1, Math.abs(e)))) {
      throw new Error(`element ${i}: got ${a}, want ${e}`);
    }
  }
}

function assertBitsEqual(actual, expected) {
  assert(actual.length === expected.length, `length ${actual.length} vs ${expected.length}`);
  const a = new Uint32Array(actual.buffer, actual.byteOffset, actual.length);
  const e = new Uint32Array(expected.buffer, expected.byteOffset, expected.length);
  for (let i = 0; i < e.length; i++) {
    if (a[i] !== e[i]) {
      throw new Error(`element ${i}: bits ${a[i].toString(16)} vs ${e[i].toString(16)} (${actual[i]} vs ${expected[i]})`);
    }
  }
}

function loadGolden(name) {
  return JSON.parse(fs.readFileSync(path.join(__dirname, '..', 'golden', name), 'utf8'));
}

/** Deterministic pseudo-random floats in [lo, hi). */
function rng(seed) {
  let s = (seed >>> 0) || 1;
  return {
    uniform(n, lo, hi) {
      const out = new Float32Array(n);
      for (let i = 0; i < n; i++) {
        s = (Math.imul(s, 1664525) + 1013904223) >>> 0;
        out[i] = lo + (s / 4294967296) * (hi - lo);
      }
      return out;
    }
  };
}

module.exports = {test, run, assert, assertEqual, assertThrows, assertClose, assertParity, assertBitsEqual, loadGolden, rng};
