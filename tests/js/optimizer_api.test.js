'use strict';
// The reference's JavaScript API for this path, driven from JavaScript: same classes, methods, argument
// order and error codes as packages/core/index.d.cts, bound to libmxopt.so by mlx-node_amd/napi/mxopt_napi.c.
// Each case names the reference test whose expectation it restates (values, digits), in this file's own words.
const { core, it, close, check, f32, run } = require('./harness');
const { Adam, AdamW, SGD, RMSprop, GradientUtils, LRScheduler, Qwen3Model, MxArray, DType } = core;

const step = (opt, name, p, g) => Array.from(opt.updateSingle(name, f32(p), f32(g)).toFloat32());

// ---- __test__/core/optimizers.test.ts -------------------------------------------------------------
it('Adam: defaults move every element down for positive gradients (:7-23)', () => {
  const v = step(new Adam(), 'param1', [1, 2, 3], [0.1, 0.2, 0.3]);
  check(v[0] < 1 && v[1] < 2 && v[2] < 3, 'smaller values');
});

it('Adam: state is per parameter name (:25-41)', () => {
  const adam = new Adam();
  const a = step(adam, 'param1', [1, 2], [0.1, 0.2]);
  const b = step(adam, 'param2', [3, 4], [0.1, 0.2]);
  check(!close(a[0], b[0]) && !close(a[1], b[1]), 'different results');
});

it('Adam: bias correction changes the first step (:43-65)', () => {
  const on = step(new Adam(0.01, 0.9, 0.999, 1e-8, true), 'param', [1, 1], [0.1, 0.1]);
  const off = step(new Adam(0.01, 0.9, 0.999, 1e-8, false), 'param', [1, 1], [0.1, 0.1]);
  check(!close(on[0], 1) && !close(off[0], 1) && !close(on[0], off[0]), 'both moved, differently');
});

it('Adam: reset() makes the next update equal to the first (:67-87)', () => {
  const adam = new Adam();
  const first = step(adam, 'param', [1, 2], [0.1, 0.2]);
  adam.reset();
  const again = step(adam, 'param', [1, 2], [0.1, 0.2]);
  check(first[0] === again[0] && first[1] === again[1], 'identical values');
});

it('Adam: a larger learning rate moves further (:89-104)', () => {
  const lo = step(new Adam(0.001), 'param', [1, 1], [0.1, 0.1]);
  const hi = step(new Adam(0.01), 'param', [1, 1], [0.1, 0.1]);
  check(Math.abs(1 - hi[0]) > Math.abs(1 - lo[0]), 'larger change');
});

it('AdamW: decoupled decay shrinks parameters that have a zero gradient (:107-130)', () => {
  const wd = step(new AdamW(0.01, 0.9, 0.999, 1e-8, 0.01), 'param', [1, 2, 3], [0, 0, 0]);
  const plain = step(new Adam(0.01, 0.9, 0.999, 1e-8), 'param', [1, 2, 3], [0, 0, 0]);
  check(wd[0] < 1 && wd[1] < 2 && wd[2] < 3, 'decayed values');
  check(close(plain[0], 1, 5) && close(plain[1], 2, 5) && close(plain[2], 3, 5), 'Adam leaves them alone');
  check(close(wd[0], 1 * (1 - 0.01 * 0.01), 6), 'p * (1 - lr*wd)');
});

it('SGD: p - lr*g (:151-164)', () => {
  const v = step(new SGD(0.1), 'param', [1, 2, 3], [0.1, 0.2, 0.3]);
  check(close(v[0], 0.99, 5) && close(v[1], 1.98, 5) && close(v[2], 2.97, 5), '[0.99, 1.98, 2.97]');
});

it('SGD: momentum 0.9, two steps (:166-188)', () => {
  const sgd = new SGD(0.1, 0.9);
  const one = sgd.updateSingle('param', f32([1, 1]), f32([0.1, 0.1]));
  check(close(one.toFloat32()[0], 0.99, 5), 'first step 0.99');
  const two = sgd.updateSingle('param', one, f32([0.1, 0.1])).toFloat32();
  check(close(two[0], 0.971, 5), 'second step 0.99 - 0.1*(0.9*0.1 + 0.1) = 0.971');
});

it('SGD: L2 weight decay is added to the gradient (:190-203)', () => {
  const v = step(new SGD(0.1, 0.0, 0.01), 'param', [1, 2], [0.1, 0.2]);
  check(close(v[0], 1 - 0.1 * (0.1 + 0.01 * 1), 5) && close(v[1], 2 - 0.1 * (0.2 + 0.01 * 2), 5), 'closed form');
});

it('SGD: Nesterov needs momentum and no dampening -> InvalidArg (:205-214)', () => {
  for (const args of [[0.1, 0.0, 0.0, 0.0, true], [0.1, 0.9, 0.0, 0.1, true]]) {
    let err = null;
    try { new SGD(...args); } catch (e) { err = e; }
    check(err && err.code === 'InvalidArg' && /Nesterov/.test(err.message), 'an InvalidArg error, got ' + err);
  }
  new SGD(0.1, 0.9, 0.0, 0.0, true);
});

it('RMSprop: moves down, alpha changes the step (:218-277)', () => {
  const a = step(new RMSprop(0.01), 'param', [1, 2, 3], [0.1, 0.2, 0.3]);
  check(a[0] < 1 && a[1] < 2 && a[2] < 3, 'smaller values');
  const hi = new RMSprop(0.01, 0.99), lo = new RMSprop(0.01, 0.5);
  let ph = f32([1, 1]), pl = f32([1, 1]);
  for (let i = 0; i < 3; i++) { ph = hi.updateSingle('param', ph, f32([0.1, 0.1])); pl = lo.updateSingle('param', pl, f32([0.1, 0.1])); }
  check(!close(ph.toFloat32()[0], pl.toFloat32()[0], 4), 'different trajectories');
});

it('GradientUtils.clipGradValue (:281-291)', () => {
  const v = GradientUtils.clipGradValue(f32([-2, -0.5, 0, 0.5, 2]), -1, 1).toFloat32();
  [-1, -0.5, 0, 0.5, 1].forEach((w, i) => check(close(v[i], w, 5), `element ${i} = ${w}`));
});

it('GradientUtils.computeGradientNorm (:293-310)', () => {
  check(close(GradientUtils.computeGradientNorm({ param1: f32([3, 4]) }), 5, 5), 'norm 5');
  check(close(GradientUtils.computeGradientNorm({ param1: f32([1, 2]), param2: f32([2]) }), 3, 5), 'norm 3');
});

it('GradientUtils.clipGradNorm (:312-351)', () => {
  const same = GradientUtils.clipGradNorm({ param: f32([3, 4]) }, 10).param.toFloat32();
  check(close(same[0], 3, 5) && close(same[1], 4, 5), 'unchanged below the limit');
  const half = GradientUtils.clipGradNorm({ param: f32([3, 4]) }, 2.5).param.toFloat32();
  check(close(half[0], 1.5, 4) && close(half[1], 2, 4), 'halved');
  const two = GradientUtils.clipGradNorm({ param1: f32([1, 2]), param2: f32([2]) }, 1.5);
  const a = two.param1.toFloat32(), b = two.param2.toFloat32();
  check(close(a[0], 0.5, 4) && close(a[1], 1, 4) && close(b[0], 1, 4), 'all tensors scaled by 0.5');
});

it('GradientUtils.clipGradNormWithNorm returns [gradients, norm] (:353-365)', () => {
  const [clipped, norm] = GradientUtils.clipGradNormWithNorm({ param: f32([3, 4]) }, 2.5);
  check(close(norm, 5, 5) && close(clipped.param.toFloat32()[0], 1.5, 4), 'norm 5 and halved values');
});

it('LRScheduler closed forms (:382-433)', () => {
  check(close(LRScheduler.linearDecay(1, 0.1, 50, 100), 0.55, 5) && LRScheduler.linearDecay(1, 0.1, 200, 100) === 0.1, 'linear');
  check(close(LRScheduler.exponentialDecay(1, 0.9, 20, 10), 0.81, 5), 'exponential');
  check(close(LRScheduler.cosineAnnealing(1, 0.1, 50, 100), 0.55, 5) && LRScheduler.cosineAnnealing(1, 0.1, 100, 100) === 0.1, 'cosine');
  check(LRScheduler.stepDecay(1, 0.5, 9, 10) === 1 && close(LRScheduler.stepDecay(1, 0.5, 30, 10), 0.125, 5), 'step');
});

it('quadratic descent converges with Adam and with SGD+momentum (:436-475)', () => {
  let x = f32([10]);
  const adam = new Adam(0.1);
  for (let i = 0; i < 100; i++) x = adam.updateSingle('x', x, f32([2 * x.toFloat32()[0]]));
  check(Math.abs(x.toFloat32()[0]) < 10, 'Adam moved towards 0');
  x = f32([10]);
  const sgd = new SGD(0.1, 0.9);
  for (let i = 0; i < 100; i++) x = sgd.updateSingle('x', x, f32([2 * x.toFloat32()[0]]));
  check(Math.abs(x.toFloat32()[0]) < 1, 'SGD+momentum close to 0');
});

// ---- __test__/trainers/grpo-gradient-accumulation.test.ts -------------------------------------------
it('Qwen3Model.accumulateGradients sums, copies new names, keeps old ones (:7-44, model.rs:2235-2240)', () => {
  const acc = Qwen3Model.accumulateGradients({ param1: f32([1, 2]), param2: f32([3]), only_old: f32([9]) },
                                             { param1: f32([0.5, 1.5]), param2: f32([1]), only_new: f32([7, 8]) });
  check(close(acc.param1.toFloat32()[0], 1.5, 5) && close(acc.param1.toFloat32()[1], 3.5, 5), 'param1 summed');
  check(close(acc.param2.toFloat32()[0], 4, 5), 'param2 summed');
  check(acc.only_new.toFloat32()[1] === 8 && acc.only_old.toFloat32()[0] === 9, 'names on one side only');
  const first = Qwen3Model.accumulateGradients({}, { param1: f32([1, 2]) });
  check(first.param1.toFloat32()[0] === 1 && first.param1.toFloat32()[1] === 2, 'first accumulation is a copy');
});

it('N identical micro-batches sum to N times the gradient, shape kept (:48-91)', () => {
  let acc = {};
  for (let i = 0; i < 4; i++) acc = Qwen3Model.accumulateGradients(acc, { weight: f32([1, 2, 3, 4], [2, 2]) });
  const v = acc.weight.toFloat32();
  [4, 8, 12, 16].forEach((w, i) => check(close(v[i], w, 5), `element ${i}`));
  check(Array.from(acc.weight.shape()).map(Number).join() === '2,2' && acc.weight.size() === 4n, 'shape [2,2]');
});

// ---- dtype surface -----------------------------------------------------------------------------------
it('bf16 arrays: astype rounds to nearest even, optimizers return float32 (adamw.rs:116)', () => {
  const x = f32([1.00390625, 1.01171875, -3.0e-5]);     // 1 + 2^-8 ties to even (1.0); 1 + 3*2^-8 ties up
  const b = x.astype(DType.BFloat16);
  check(b.dtype() === DType.BFloat16 && x.dtype() === DType.Float32, 'dtype codes 3 and 0');
  const back = Array.from(b.toFloat32());
  check(back[0] === 1.0 && back[1] === 1.015625, 'ties to even: ' + back);
  const out = new AdamW(0.01).updateSingle('w', b, f32([0.1, 0.1, 0.1]).astype(DType.BFloat16));
  check(out.dtype() === DType.Float32 && out.toFloat32()[0] < 1.0, 'float32 result');
  check(MxArray.zeros([2, 3], DType.Float16).toFloat32().every((v) => v === 0), 'zeros');
});

it('wrong argument types are refused with InvalidArg', () => {
  let err = null;
  try { new Adam().updateSingle('p', { not: 'an array' }, f32([1])); } catch (e) { err = e; }
  check(err && err.code === 'InvalidArg', 'InvalidArg, got ' + err);
  err = null;
  try { new Adam().updateSingle('p', f32([1, 2]), f32([1])); } catch (e) { err = e; }
  check(err && err.code === 'InvalidArg', 'size mismatch refused, got ' + err);
});

run();
