// Drives the Node-API addon (framework_amd/lib/mni_rocm.node) the way the
// reference's TypeScript layer drives its native addon: a Tensor class that
// only forwards ids (cf. src/tensor.ts), Linear / mseLoss / Adam on top of it
// (cf. src/nn.ts, src/optimizer.ts), and the assertions the reference's own
// suite makes about the matmul path (test/tensor.test.ts MatMul section,
// test/autograd.test.ts, test/nn.test.ts, test/module.test.ts).  Needs a GPU.
'use strict';
const path = require('path');
const native = require(path.join(__dirname, '..', '..', 'framework_amd', 'lib', 'mni_rocm.node'));

let passed = 0, failed = 0;
function assert(cond, msg) { if (cond) { passed++; } else { failed++; console.log('FAIL: ' + msg); } }
function assertClose(a, b, tol, msg) { assert(Math.abs(a - b) <= tol, msg + ' (got ' + a + ', want ' + b + ')'); }

class Tensor {
  constructor(id, shape) { this._id = id; this._shape = shape || native.tensorShape(id).map(Number); }
  get shape() { return this._shape; }
  get grad() { const g = native.getGrad(this._id); return g == null ? null : new Tensor(g); }
  static fromFloat32(data, shape) { return new Tensor(native.fromFloat32(data, shape), shape); }
  toFloat32() { return native.toFloat32(this._id); }
  setRequiresGrad(r) { native.setRequiresGrad(this._id, r); return this; }
  matmul(o) { return new Tensor(native.matmul(this._id, o._id)); }
  add(o) { return new Tensor(native.add(this._id, o._id)); }
  sub(o) { return new Tensor(native.sub(this._id, o._id)); }
  mul(o) { return typeof o === 'number' ? new Tensor(native.mulScalar(this._id, o)) : new Tensor(native.mul(this._id, o._id)); }
  relu() { return new Tensor(native.relu(this._id)); }
  sum(dim) { return new Tensor(dim === undefined ? native.sumAll(this._id) : native.sumOp(this._id, dim)); }
  permute(...dims) { return new Tensor(native.permute(this._id, dims)); }
  backward() { native.backward(this._id); }
}
function lcg(seed) { let s = seed >>> 0; return () => { s = (Math.imul(s, 1664525) + 1013904223) >>> 0; return s / 4294967296; }; }
function randArray(n, rnd, lo, hi) { const a = new Float32Array(n); for (let i = 0; i < n; i++) a[i] = lo + (hi - lo) * rnd(); return a; }
class Linear {
  constructor(inF, outF, rnd, fused) {
    const b = 1 / Math.sqrt(inF);
    this.weight = Tensor.fromFloat32(randArray(inF * outF, rnd, -b, b), [inF, outF]).setRequiresGrad(true);
    this.bias = Tensor.fromFloat32(randArray(outF, rnd, -b, b), [outF]).setRequiresGrad(true);
    this.fused = fused && typeof native.linear === 'function';   // the reference's feature-detection idiom
  }
  forward(x) {
    if (this.fused) return new Tensor(native.linear(x._id, this.weight._id, this.bias._id, 1));
    return x.matmul(this.weight).add(this.bias);
  }
  parameters() { return [this.weight, this.bias]; }
}
function mseLoss(pred, target) {  // mean(-1) twice, as the reference does
  const d = pred.sub(target); const sq = d.mul(d);
  return new Tensor(native.meanOp(native.meanOp(sq._id, -1), -1));
}

// ---- MatMul (test/tensor.test.ts) ------------------------------------------------------
const mm = Tensor.fromFloat32(new Float32Array([1, 2, 3, 4]), [2, 2]).matmul(Tensor.fromFloat32(new Float32Array([5, 6, 7, 8]), [2, 2])).toFloat32();
assertClose(mm[0], 19, 1e-3, 'matmul [0,0]'); assertClose(mm[1], 22, 1e-3, 'matmul [0,1]');
assertClose(mm[2], 43, 1e-3, 'matmul [1,0]'); assertClose(mm[3], 50, 1e-3, 'matmul [1,1]');
const ns = Tensor.fromFloat32(new Float32Array([1, 2, 3, 4, 5, 6]), [2, 3]).matmul(Tensor.fromFloat32(new Float32Array([1, 2, 3, 4, 5, 6]), [3, 2]));
assert(ns.shape[0] === 2 && ns.shape[1] === 2, 'matmul [2,3]x[3,2] -> [2,2]');
assertClose(ns.toFloat32()[0], 22, 1e-3, 'matmul non-square [0,0]');
const rnd = lcg(7);
const bm = Tensor.fromFloat32(randArray(60, rnd, 0, 1), [4, 3, 5]).matmul(Tensor.fromFloat32(randArray(40, rnd, 0, 1), [4, 5, 2]));
assert(bm.shape.join() === '4,3,2', 'batched matmul shape');

// ---- a larger product against a JS triple loop, through a permuted view ---------------
{
  const M = 70, K = 45, N = 90;
  const a = randArray(M * K, rnd, -1, 1), bt = randArray(N * K, rnd, -1, 1);  // bt is B^T, viewed through permute
  const got = Tensor.fromFloat32(a, [M, K]).matmul(Tensor.fromFloat32(bt, [N, K]).permute(1, 0)).toFloat32();
  let worst = 0;
  for (let i = 0; i < M; i++) for (let j = 0; j < N; j++) {
    let s = 0; for (let k = 0; k < K; k++) s += a[i * K + k] * bt[j * K + k];
    worst = Math.max(worst, Math.abs(s - got[i * N + j]));
  }
  assert(worst <= 1e-4 * Math.sqrt(K), 'permuted-view matmul vs JS loop, max err ' + worst);
}

// ---- autograd through matmul (test/autograd.test.ts) -------------------------------------
const mmX = Tensor.fromFloat32(new Float32Array([1, 0, 0, 1]), [2, 2]).setRequiresGrad(true);
const mmY = Tensor.fromFloat32(new Float32Array([3, 4, 5, 6]), [2, 2]).setRequiresGrad(true);
mmX.matmul(mmY).sum().backward();
assert(mmX.grad !== null, 'matmul grad exists');
assert(Array.from(mmX.grad.toFloat32()).join() === '7,11,7,11', 'dX = G Y^T');
assert(Array.from(mmY.grad.toFloat32()).join() === '1,1,1,1', 'dY = X^T G');

// ---- Linear and losses (test/nn.test.ts) ------------------------------------------------------
for (const fused of [false, true]) {
  const lin = new Linear(3, 2, lcg(3), fused);
  const out = lin.forward(Tensor.fromFloat32(randArray(12, rnd, 0, 1), [4, 3]));
  assert(out.shape[0] === 4 && out.shape[1] === 2, 'linear [4,3] -> [4,2] fused=' + fused);
  assert(lin.parameters().length === 2, 'linear has weight + bias');
}
const p = Tensor.fromFloat32(new Float32Array([1, 2, 3, 4]), [2, 2]);
assertClose(mseLoss(p, Tensor.fromFloat32(new Float32Array([1, 2, 3, 4]), [2, 2])).toFloat32()[0], 0, 1e-4, 'mseLoss identical = 0');
assertClose(mseLoss(p, Tensor.fromFloat32(new Float32Array([2, 3, 4, 5]), [2, 2])).toFloat32()[0], 1.0, 1e-4, 'mseLoss off-by-1 = 1.0');

// ---- end-to-end regression (test/module.test.ts) --------------------------------------------------
{
  const X = Tensor.fromFloat32(new Float32Array([0, 1, 2, 3, 4, 5]), [6, 1]);
  const Y = Tensor.fromFloat32(new Float32Array([1, 3, 5, 7, 9, 11]), [6, 1]);
  const net = new Linear(1, 1, lcg(11), false);
  const ids = net.parameters().map(t => t._id);
  let early = null, t = 0;
  for (let i = 0; i < 200; i++) {
    native.zeroGrad(ids);
    const loss = mseLoss(net.forward(X), Y);
    if (i === 10) early = loss.toFloat32()[0];
    loss.backward();
    native.clipAndStep(ids, 0.05, 0.9, 0.95, 1e-8, 0, ++t, 0);   // Adam {lr: 0.05}
    native.gcTensors([X._id, Y._id].concat(ids, ids.map(id => native.getGrad(id))));
  }
  const final = mseLoss(net.forward(X), Y).toFloat32()[0];
  assert(final < early, 'training reduces loss'); assert(final < 1.0, 'training converges to low loss (' + final + ')');
}

// ---- softmax / flashAttention (test/nn.test.ts:46-54, test/native.test.ts:13-23) -----------------------
{
  const sm = native.toFloat32(native.softmaxOp(Tensor.fromFloat32(new Float32Array([1, 2, 3, 1, 2, 3]), [2, 3])._id, 1));
  assertClose(sm[0] + sm[1] + sm[2], 1.0, 1e-4, 'softmax row0 sums to 1');
  assertClose(sm[3] + sm[4] + sm[5], 1.0, 1e-4, 'softmax row1 sums to 1');
  assert(sm.every(v => v > 0) && sm[2] > sm[1] && sm[1] > sm[0], 'softmax positive and ordered');
  const bg = new Tensor(native.biasGelu(Tensor.fromFloat32(randArray(8, rnd, 0, 1), [2, 4])._id, Tensor.fromFloat32(randArray(4, rnd, 0, 1), [4])._id));
  assert(bg.shape[0] === 2 && bg.shape[1] === 4, 'biasGelu shape');   // test/native.test.ts:39-43
  assert(typeof native.flashAttention === 'function', 'flashAttention is exported');
  const nHeads = 2, seqLen = 4, headDim = 8;
  const mk = () => Tensor.fromFloat32(randArray(nHeads * seqLen * headDim, rnd, 0, 1), [nHeads, seqLen, headDim]);
  const q = mk(), k = mk(), v = mk();
  const att = new Tensor(native.flashAttention(q._id, k._id, v._id, 1.0 / Math.sqrt(headDim), true));
  assert(att.shape.join() === [nHeads, seqLen, headDim].join(), 'attention output shape');
  const a = att.toFloat32(), vv = v.toFloat32();
  let worst = 0;  // causal row 0 attends to key 0 only
  for (let h = 0; h < nHeads; h++) for (let d = 0; d < headDim; d++) worst = Math.max(worst, Math.abs(a[h * seqLen * headDim + d] - vv[h * seqLen * headDim + d]));
  assert(worst < 1e-6, 'causal attention row 0 equals v[0]');
}

// ---- KV cache (test/native.test.ts:48-151) -----------------------------------------------------------
{
  const batch = 1, heads = 2, headDim = 8, maxSeq = 16, steps = 6, scale = 1 / Math.sqrt(headDim);
  const mk = (s) => Tensor.fromFloat32(randArray(batch * heads * s * headDim, rnd, 0, 1), [batch, heads, s, headDim]);
  const fp = native.kvCacheCreate(batch, heads, headDim, maxSeq, false), qc = native.kvCacheCreate(batch, heads, headDim, maxSeq, true);
  assert(native.kvCacheQuantized(qc) === true && native.kvCacheQuantized(fp) === false, 'quantized flag');
  let maxAbsDiff = 0;
  for (let t = 0; t < steps; t++) {
    const q = mk(1), k = mk(1), v = mk(1);
    const a = native.toFloat32(native.kvCacheDecodeStep(fp, q._id, k._id, v._id, scale));
    const b = native.toFloat32(native.kvCacheDecodeStep(qc, q._id, k._id, v._id, scale));
    for (let i = 0; i < a.length; i++) maxAbsDiff = Math.max(maxAbsDiff, Math.abs(a[i] - b[i]));
    assert(a.length === batch * heads * headDim, 'decode output size');
  }
  assert(Number(native.kvCacheLen(fp)) === steps && Number(native.kvCacheLen(qc)) === steps, 'kv cache length tracks decode steps');
  assert(maxAbsDiff < 0.15, 'quantized kv decode drift bounded (' + maxAbsDiff.toFixed(4) + ')');
  let threw = false;
  try { const t2 = mk(2); native.kvCacheDecodeStep(fp, t2._id, t2._id, t2._id, scale); } catch (e) { threw = /seq_len=1/.test(e.message); }
  assert(threw, 'decode step rejects seq_len != 1');
  const small = native.kvCacheCreate(batch, heads, headDim, 2, false);
  native.kvCacheAppend(small, mk(1)._id, mk(1)._id); native.kvCacheAppend(small, mk(1)._id, mk(1)._id);
  threw = false;
  try { native.kvCacheAppend(small, mk(1)._id, mk(1)._id); } catch (e) { threw = /kv cache is full/.test(e.message); }
  assert(threw, 'append rejects capacity overflow');
  native.kvCacheReset(fp);
  assert(Number(native.kvCacheLen(fp)) === 0, 'kv cache reset clears logical length');
  native.kvCacheFree(fp);
  threw = false;
  try { native.kvCacheDecodeStep(fp, mk(1)._id, mk(1)._id, mk(1)._id, scale); } catch (e) { threw = /invalid kv cache id/.test(e.message); }
  assert(threw, 'free invalidates kv cache handle');
}

// ---- token-side ops (test/nn.test.ts:176-251, test/native.test.ts:28-36) --------------------------------
{
  native.seed(7);
  const w = native.philoxWords(0, 0, 4);
  assert(w[0] === 0x6627e8d5 && w[3] === 0x9b00dbd8, 'philox known answer');
  const r = native.toFloat32(native.randTensor([1000]));
  assert(r.every(v => v >= 0 && v < 1), 'rand in [0, 1)');
  const z = native.toFloat32(native.randnTensor([4000]));
  let m = 0; for (const v of z) m += v / z.length;
  assert(Math.abs(m) < 0.1, 'randn mean near 0');
  const tiled = new Tensor(native.tile(Tensor.fromFloat32(new Float32Array([1, 2, 3]), [1, 3])._id, [2, 1]));
  const td = tiled.toFloat32();
  assert(tiled.shape[0] === 2 && tiled.shape[1] === 3 && td[0] === 1 && td[3] === 1 && td[5] === 3, 'tile [1,3] x [2,1]');
  const weight = Tensor.fromFloat32(randArray(40, rnd, -0.5, 0.5), [10, 4]).setRequiresGrad(true);
  const emb = new Tensor(native.embeddingForward(weight._id, [0, 1, 2, 3, 4, 5], 2, 3));
  assert(emb.shape.join() === '2,3,4', 'embedding shape');
  const same = native.toFloat32(native.embeddingForward(weight._id, [0, 0, 0, 0], 2, 2));
  assert(same[0] === same[4], 'same index = same embedding');
  let threw = false;
  try { native.embeddingForward(weight._id, [10], 1, 1); } catch (e) { threw = /out of range/.test(e.message); }
  assert(threw, 'embedding index out of range throws');
  const x4 = Tensor.fromFloat32(new Float32Array([1, 2, 3, 4]), [4]);
  assert(native.dropoutOp(x4._id, 0.5, false) === x4._id && native.dropoutOp(x4._id, 0.0, true) === x4._id, 'dropout passthrough');
  const dropped = native.toFloat32(native.dropoutOp(native.ones([1000]), 0.5, true));
  const zeros = dropped.filter(v => v === 0).length;
  assert(zeros > 100 && zeros < 900 && dropped.every(v => v === 0 || v === 2), 'dropout rate 0.5');
  const rln = new Tensor(native.residualLayernorm(native.randTensor([2, 4]), native.randTensor([2, 4]), native.ones([4]), native.zeros([4]), 1e-5));
  const rd = rln.toFloat32();
  assert(rln.shape.join() === '2,4' && Math.abs(rd[0] + rd[1] + rd[2] + rd[3]) < 1e-4, 'residualLayernorm rows have zero mean');
  const data = new Int32Array(500); for (let i = 0; i < 500; i++) data[i] = i % 10;
  const ds = native.createDataset(data);
  const [inp, tgt] = native.sampleBatch(ds, 8, 4);
  const a = native.intBufferToInt32(inp), b = native.intBufferToInt32(tgt);
  let ok = a.length === 32 && b.length === 32;
  for (let i = 0; i < 32; i++) ok = ok && b[i] === (a[i] + 1) % 10;
  assert(ok, 'sampleBatch targets are the inputs shifted by one');
  const e2 = new Tensor(native.embeddingForwardGpu(weight._id, inp, 4, 8));
  const logits = e2.matmul(Tensor.fromFloat32(randArray(40, rnd, -0.5, 0.5), [4, 10]));
  const loss = new Tensor(native.crossEntropyLossGpu(logits._id, tgt));
  loss.mul(1024).backward();
  assert(native.scaleGrads([weight._id], 1 / 1024) === false, 'scaleGrads reports finite gradients');
  assert(Math.abs(loss.toFloat32()[0] - Math.log(10)) < 0.5, 'cross-entropy on buffered targets near ln(10)');
  native.freeIntBuffer(inp); native.freeIntBuffer(tgt);
  threw = false;
  try { native.intBufferToInt32(inp); } catch (e) { threw = /int buffer already freed/.test(e.message); }
  assert(threw, 'freed int buffer is rejected');
}

// ---- misuse raises a JS Error where the reference panics ---------------------------------------------
try { Tensor.fromFloat32(new Float32Array(6), [2, 3]).matmul(Tensor.fromFloat32(new Float32Array(8), [4, 2])); assert(false, 'K mismatch must throw'); }
catch (e) { assert(/inner dimensions/.test(e.message), 'K mismatch message: ' + e.message); }

console.log(passed + ' passed, ' + failed + ' failed');
process.exit(failed ? 1 : 0);
