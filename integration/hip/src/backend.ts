/**
 * HipBackend: alpha2's `Backend` (packages/core/src/interfaces.ts:38-151) on libalpha_hip.so.
 *
 * Same members, argument order, shape rules and error wording as alpha2_amd/backend.py::HipBackend, which is this class
 * in the one host language the build image has and is what the parity tests drive.  Tensors are lazy like the Vulkan
 * backend's (packages/helios/src/backend.ts:1143-1171): an op returns a handle whose `.data` getter reads the device
 * buffer back on first use and caches it; in-place ops drop the cache (backend.ts:706-729); `reshape` shares the buffer
 * with a reference count (backend.ts:4528-4538).  Frees are stream-ordered in the library, so `releaseGpuTensor` may
 * free right after the last use has been enqueued.
 */
import type { Backend, Dtype, Shape, TensorArray, TensorData } from "@alpha/core";
import { SeededRng, dtypeArray, shapeSize } from "@alpha/core";
import { Bin, Dt, Epi, Layout, Struct, Un, UnBwd, addressOf, check, i64s, lib } from "./ffi.js";

const DT_CODE: Record<string, number> = { f32: Dt.F32, i32: Dt.I32, f16: Dt.F16 };
const DT_BYTES: Record<string, number> = { f32: 4, i32: 4, f16: 2, f64: 8 };

/** One ah_alloc block, shared by views. */
class Buf {
  refs = 1;
  ptr: bigint;
  constructor(readonly nbytes: number) {
    const out = new BigUint64Array(1);
    check(lib.ah_alloc(BigInt(Math.max(1, nbytes)), addressOf(out)));
    this.ptr = out[0];
  }
  release(): void {
    if (--this.refs === 0 && this.ptr !== 0n) { lib.ah_free(this.ptr); this.ptr = 0n; }
  }
}

/** Backstop for tensors the caller drops without releasing (packages/helios/src/backend.ts:627-639). */
const cleanup = new FinalizationRegistry<Buf>((buf) => {
  try { if (buf.ptr !== 0n && buf.refs > 0) { lib.ah_free(buf.ptr); buf.ptr = 0n; } } catch { /* library shut down */ }
});

/** A device-resident tensor: `.data` is fetched on demand. */
class DeviceTensor implements TensorData {
  host: TensorArray | null = null;
  constructor(readonly shape: Shape, readonly dtype: Dtype, public buf: Buf | null, public off: number, private owner: HipBackend) {}
  get data(): TensorArray {
    if (this.host === null) {
      if (this.buf === null) throw new Error("TensorData has neither host nor device contents (released?)");
      this.host = this.owner.readback(this);
    }
    return this.host;
  }
  get size(): number { return shapeSize(this.shape); }
}

interface Residency { buf: Buf; off: number }

export interface HipDeviceInfo {
  deviceName: string; arch: string; vendorId: number; computeUnits: number; waveSize: number; clockKHz: number; hbmBytes: bigint;
}

const STEP_HOW = ["eager", "recorded", "replayed", "fell-back"] as const;

export class HipBackend implements Backend {
  readonly name = "hip";
  /** Host-created tensors (plain objects from loaders, `fromArray`, `randn`) that have been uploaded, by identity. */
  private uploaded = new WeakMap<TensorData, Residency>();
  private rng: SeededRng | null = null;
  private hyper: Buf | null = null;
  private hyperKey = "";
  private gemmDesc = new Struct("AhGemm");
  private flashDesc = new Struct("AhFlash");
  private adamDesc = new Struct("AhAdamW");
  private stepGraphs = false;
  private stepOpen = false;
  private stepKey = 0n;
  lastStepHow: (typeof STEP_HOW)[number] = "eager";
  lastStepNote = "";

  constructor(device = 0) { check(lib.ah_init(device)); }

  // ── residency ────────────────────────────────────────────────────────────
  private alloc(shape: Shape, dtype: Dtype = "f32"): DeviceTensor {
    const buf = new Buf(shapeSize(shape) * DT_BYTES[dtype]);
    const t = new DeviceTensor([...shape], dtype, buf, 0, this);
    cleanup.register(t, buf, t);
    return t;
  }

  /** Device address of `t`; a host-created tensor is uploaded on first use. */
  private h(t: TensorData): bigint {
    if (t instanceof DeviceTensor) {
      if (t.buf === null) throw new Error("use of a released tensor");
      return t.buf.ptr + BigInt(t.off);
    }
    let r = this.uploaded.get(t);
    if (r === undefined) {
      const host = t.data;
      const buf = new Buf(host.byteLength);
      if (host.byteLength > 0) check(lib.ah_upload(buf.ptr, addressOf(host), BigInt(host.byteLength)));
      r = { buf, off: 0 };
      this.uploaded.set(t, r);
      cleanup.register(t, buf, t);
    }
    return r.buf.ptr + BigInt(r.off);
  }

  readback(t: DeviceTensor): TensorArray {
    const n = shapeSize(t.shape);
    const out = new (dtypeArray(t.dtype))(n);
    if (n > 0) check(lib.ah_download(addressOf(out), t.buf!.ptr + BigInt(t.off), BigInt(out.byteLength)));   // blocks
    return out;
  }

  /** An in-place device op changed `t`: its cached host copy is stale. */
  private dirty(t: TensorData): void {
    if (t instanceof DeviceTensor) t.host = null;
  }

  private view(t: TensorData, shape: Shape): DeviceTensor {
    this.h(t);
    const r: Residency = t instanceof DeviceTensor ? { buf: t.buf!, off: t.off } : this.uploaded.get(t)!;
    r.buf.refs++;
    const v = new DeviceTensor([...shape], t.dtype, r.buf, r.off, this);
    cleanup.register(v, r.buf, v);
    return v;
  }

  private static f32(...ts: TensorData[]): void {
    for (const t of ts) if (t.dtype !== "f32") throw new TypeError(`op expects f32 tensors, got ${t.dtype}`);
  }

  /** The data-movement kernels copy 4-byte elements. */
  private static words(...ts: TensorData[]): void {
    for (const t of ts) if (DT_BYTES[t.dtype] !== 4) throw new TypeError(`data-movement op expects 4-byte storage, got ${t.dtype}`);
  }

  private static axis(axis: number, nd: number): number {
    const a = axis < 0 ? axis + nd : axis;
    if (a < 0 || a >= nd) throw new Error(`axis ${axis} out of range for ndim ${nd}`);
    return a;
  }

  // ── duck-typed members the trainer probes for (packages/train/src/trainer.ts:1003-1032,1915) ─────────────
  releaseGpuTensor(t: TensorData): void {
    if (t instanceof DeviceTensor) {
      if (t.buf === null) return;
      cleanup.unregister(t);
      t.buf.release();
      t.buf = null;
      return;
    }
    const r = this.uploaded.get(t);
    if (r !== undefined) { cleanup.unregister(t); r.buf.release(); this.uploaded.delete(t); }
  }

  /** The trainer's end-of-step call (trainer.ts:1776-1784).  Work is already on the stream in call order; with step
   *  graphs enabled this is the seam between two steps: the open step plan is closed and the next one opened. */
  flush(): void {
    if (!this.stepGraphs) return;
    if (this.stepOpen) this.stepEnd();
    this.stepBegin();
  }
  enableStepGraphs(on = true, key = 0): void {
    if (!on && this.stepOpen) this.stepEnd();
    this.stepGraphs = on;
    this.stepKey = BigInt(key);
  }
  stepBegin(): void { check(lib.ah_step_begin(this.stepKey)); this.stepOpen = true; }
  stepEnd(): string {
    const how = new Int32Array(1);
    this.stepOpen = false;
    check(lib.ah_step_end(addressOf(how)));
    this.lastStepHow = STEP_HOW[how[0]];
    this.lastStepNote = String(lib.ah_step_note());
    return this.lastStepHow;
  }
  resetStepPlan(): void { check(lib.ah_step_reset(this.stepKey)); }
  syncGpu(): void { check(lib.ah_sync()); }
  purgeBufferPools(): void { check(lib.ah_trim_pool()); }
  resetStepOps(): void { check(lib.ah_reset_op_count()); }
  get gpuOpsThisStep(): number { return Number(this.stats().getU64("ops_launched")); }

  private stats(): Struct<"AhStats"> {
    const s = new Struct("AhStats");
    check(lib.ah_stats(s.p));
    return s;
  }

  /** The fields read at packages/train/src/trainer.ts:1821-1843,1922-1930. */
  gpuMemStats(): Record<string, number> {
    const s = this.stats();
    const n = (f: string) => Number(s.getU64(f));
    return {
      bufferPoolEntries: n("pool_blocks"), bufferPoolBytes: n("pool_bytes"), outputPoolEntries: 0, outputPoolBytes: 0,
      deferredReleases: 0, pendingDestroys: 0, liveAllocs: n("live_allocs"), liveBytes: n("live_bytes"),
      totalAllocs: n("device_mallocs"), graphsLive: n("graphs_live"),
    };
  }

  getDeviceInfo(): HipDeviceInfo {
    const d = new Struct("AhDeviceInfo");
    check(lib.ah_device_info(d.p));
    return {
      deviceName: d.getString("name", 128), arch: d.getString("arch", 32), vendorId: 0x1002, computeUnits: d.getI32("compute_units"),
      waveSize: d.getI32("wavefront"), clockKHz: d.getI32("clock_khz"), hbmBytes: d.getU64("hbm_bytes"),
    };
  }

  setMinGpuSize(_n: number): void { /* every op runs on the device; kept for interface compatibility */ }

  // ── creation ────────────────────────────────────────────────────────────
  zeros(shape: Shape, dtype: Dtype = "f32"): TensorData { return this.full(shape, 0, dtype); }
  ones(shape: Shape, dtype: Dtype = "f32"): TensorData { return this.full(shape, 1, dtype); }
  full(shape: Shape, value: number, dtype: Dtype = "f32"): TensorData {
    const t = this.alloc(shape, dtype);
    const n = BigInt(shapeSize(shape));
    if (dtype === "i32") check(lib.ah_fill_i32(t.buf!.ptr, Math.trunc(value), n));
    else if (dtype === "f32") check(lib.ah_fill_f32(t.buf!.ptr, value, n));
    else throw new Error(`full: dtype ${dtype} not supported`);
    return t;
  }
  randn(shape: Shape, dtype: Dtype = "f32"): TensorData {
    this.rng ??= new SeededRng(42);                                  // packages/tensor/src/cpu_ref.ts:111
    const out = new (dtypeArray(dtype))(shapeSize(shape));
    for (let i = 0; i < out.length; i++) out[i] = this.rng.nextGauss();
    return { shape: [...shape], dtype, data: out };
  }
  fromArray(data: number[], shape: Shape, dtype: Dtype = "f32"): TensorData {
    if (data.length !== shapeSize(shape)) throw new Error(`Data length ${data.length} does not match shape size ${shapeSize(shape)}`);
    return { shape: [...shape], dtype, data: (dtypeArray(dtype) as any).from(data) };
  }

  // ── math ────────────────────────────────────────────────────────────────
  private static bstrides(src: readonly number[], target: readonly number[]): number[] {
    const st = new Array<number>(target.length).fill(0);
    let s = 1;
    for (let i = target.length - 1; i >= 0; i--) { st[i] = src[i] === 1 && target[i] !== 1 ? 0 : s; s *= src[i]; }
    return st;
  }

  private binary(op: number, a: TensorData, b: TensorData): TensorData {
    HipBackend.f32(a, b);
    const same = a.shape.length === b.shape.length && a.shape.every((d, i) => d === b.shape[i]);
    if (same) {
      const out = this.alloc(a.shape);
      check(lib.ah_binary(op, this.h(a), this.h(b), out.buf!.ptr, BigInt(shapeSize(a.shape))));
      return out;
    }
    const nd = Math.max(a.shape.length, b.shape.length);
    const sa = [...new Array(nd - a.shape.length).fill(1), ...a.shape];
    const sb = [...new Array(nd - b.shape.length).fill(1), ...b.shape];
    const res: number[] = [];
    for (let i = 0; i < nd; i++) {
      if (sa[i] !== sb[i] && sa[i] !== 1 && sb[i] !== 1) throw new Error(`Cannot broadcast shapes [${a.shape}] and [${b.shape}]`);
      res.push(Math.max(sa[i], sb[i]));
    }
    if (nd > 6) throw new Error("broadcast over more than 6 dims is not supported");
    const out = this.alloc(res);
    check(lib.ah_binary_broadcast(op, this.h(a), this.h(b), out.buf!.ptr, nd, addressOf(i64s(res)),
      addressOf(i64s(HipBackend.bstrides(sa, res))), addressOf(i64s(HipBackend.bstrides(sb, res)))));
    return out;
  }
  add(a: TensorData, b: TensorData): TensorData { return this.binary(Bin.ADD, a, b); }
  sub(a: TensorData, b: TensorData): TensorData { return this.binary(Bin.SUB, a, b); }
  mul(a: TensorData, b: TensorData): TensorData { return this.binary(Bin.MUL, a, b); }
  div(a: TensorData, b: TensorData): TensorData { return this.binary(Bin.DIV, a, b); }

  private gemm(layout: number, a: bigint, b: bigint, c: bigint, m: number, n: number, k: number, lda: number, ldb: number, ldc: number,
               batch = 1, sa = 0, sb = 0, sc = 0, inDt: number = Dt.F32, outDt: number = Dt.F32, epi: number = Epi.NONE, aux = 0n): void {
    const g = this.gemmDesc;
    g.i32("layout", layout).i32("in_dtype", inDt).i32("out_dtype", outDt).i32("epilogue", epi);
    g.i64("m", m).i64("n", n).i64("k", k).i64("lda", lda).i64("ldb", ldb).i64("ldc", ldc);
    g.i64("batch", batch).i64("stride_a", sa).i64("stride_b", sb).i64("stride_c", sc);
    g.u64("a", a).u64("b", b).u64("c", c).u64("aux", aux);
    check(lib.ah_gemm(g.p));
  }

  /** Broadcast batch dims (packages/tensor/src/cpu_ref.ts:184-243): one uniform stride per operand, or null. */
  private static batched(a: TensorData, b: TensorData, aMat: number, bMat: number): { bs: number[]; batch: number; sa: number | null; sb: number | null } {
    const aB = a.shape.slice(0, -2), bB = b.shape.slice(0, -2);
    const nb = Math.max(aB.length, bB.length);
    const pa = [...new Array(nb - aB.length).fill(1), ...aB], pb = [...new Array(nb - bB.length).fill(1), ...bB];
    const bs: number[] = [];
    for (let i = 0; i < nb; i++) {
      if (pa[i] !== pb[i] && pa[i] !== 1 && pb[i] !== 1) throw new Error(`matmul batch shape mismatch: [${a.shape}] x [${b.shape}]`);
      bs.push(Math.max(pa[i], pb[i]));
    }
    const batch = shapeSize(bs), eq = (x: number[], y: number[]) => x.every((d, i) => d === y[i]);
    if (batch === 1) return { bs, batch: 1, sa: 0, sb: 0 };
    if (eq(pa, bs) && eq(pb, bs)) return { bs, batch, sa: aMat, sb: bMat };
    if (shapeSize(pa) === 1 && eq(pb, bs)) return { bs, batch, sa: 0, sb: bMat };
    if (shapeSize(pb) === 1 && eq(pa, bs)) return { bs, batch, sa: aMat, sb: 0 };
    return { bs, batch, sa: null, sb: null };
  }

  matmul(a: TensorData, b: TensorData): TensorData {
    HipBackend.f32(a, b);
    if (a.shape.length < 2 || b.shape.length < 2) throw new Error(`matmul requires at least 2D tensors, got [${a.shape}] x [${b.shape}]`);
    const M = a.shape.at(-2)!, K = a.shape.at(-1)!, N = b.shape.at(-1)!;
    if (b.shape.at(-2) !== K) throw new Error(`matmul shape mismatch: [${a.shape}] x [${b.shape}]`);
    let { bs, batch, sa, sb } = HipBackend.batched(a, b, M * K, K * N);
    if (sa === null || sb === null) {                                // mixed broadcast: materialise the operands first
      if (a.shape.length - 2 !== bs.length || !bs.every((d, i) => d === a.shape[i])) a = this.broadcast(a, [...bs, M, K]);
      if (b.shape.length - 2 !== bs.length || !bs.every((d, i) => d === b.shape[i])) b = this.broadcast(b, [...bs, K, N]);
      sa = M * K; sb = K * N;
    }
    const out = this.alloc([...bs, M, N]);
    this.gemm(Layout.NN, this.h(a), this.h(b), out.buf!.ptr, M, N, K, K, N, N, batch, sa, sb, M * N);
    return out;
  }

  /** A[.., M, K] x B[.., N, K]^T (interfaces.ts:111). */
  matmulTransposed(a: TensorData, b: TensorData): TensorData {
    HipBackend.f32(a, b);
    const M = a.shape.at(-2)!, K = a.shape.at(-1)!, N = b.shape.at(-2)!;
    if (b.shape.at(-1) !== K) throw new Error(`matmul shape mismatch: [${a.shape}] x [${b.shape}]^T`);
    const { bs, batch, sa, sb } = HipBackend.batched(a, b, M * K, N * K);
    if (sa === null || sb === null) throw new Error("matmulTransposed: mixed batch broadcast is not supported");
    const out = this.alloc([...bs, M, N]);
    this.gemm(Layout.NT, this.h(a), this.h(b), out.buf!.ptr, M, N, K, K, K, N, batch, sa, sb, M * N);
    return out;
  }

  /** A[.., M, K]^T x B[.., M, N] -> [.., K, N] (interfaces.ts:112). */
  matmulTransposedA(a: TensorData, b: TensorData): TensorData {
    HipBackend.f32(a, b);
    const M = a.shape.at(-2)!, K = a.shape.at(-1)!, N = b.shape.at(-1)!;
    if (b.shape.at(-2) !== M) throw new Error(`matmul shape mismatch: [${a.shape}]^T x [${b.shape}]`);
    const { bs, batch, sa, sb } = HipBackend.batched(a, b, M * K, M * N);
    if (sa === null || sb === null) throw new Error("matmulTransposedA: mixed batch broadcast is not supported");
    const out = this.alloc([...bs, K, N]);
    this.gemm(Layout.TN, this.h(a), this.h(b), out.buf!.ptr, K, N, M, K, N, N, batch, sa, sb, K * N);   // contraction length M
    return out;
  }

  sum(a: TensorData, axis?: number, keepdims = false): TensorData { return this.reduce(a, axis, keepdims, 0); }
  mean(a: TensorData, axis?: number, keepdims = false): TensorData { return this.reduce(a, axis, keepdims, 1); }
  private reduce(a: TensorData, axis: number | undefined, keepdims: boolean, mean: number): TensorData {
    HipBackend.f32(a);
    if (axis === undefined) {
      const out = this.alloc(keepdims ? a.shape.map(() => 1) : []);
      check(lib.ah_sum_all(this.h(a), out.buf!.ptr, BigInt(shapeSize(a.shape)), mean));
      return out;
    }
    const ax = HipBackend.axis(axis, a.shape.length);
    const outer = shapeSize(a.shape.slice(0, ax)), dim = a.shape[ax], inner = shapeSize(a.shape.slice(ax + 1));
    const oshape = keepdims ? a.shape.map((d, i) => (i === ax ? 1 : d)) : a.shape.filter((_, i) => i !== ax);
    const out = this.alloc(oshape);
    check(lib.ah_sum_axis(this.h(a), out.buf!.ptr, BigInt(outer), BigInt(dim), BigInt(inner), mean));
    return out;
  }

  // ── element-wise ────────────────────────────────────────────────────────
  private unary(op: number, a: TensorData, p0 = 0, p1 = 0): TensorData {
    HipBackend.f32(a);
    const out = this.alloc(a.shape);
    check(lib.ah_unary(op, this.h(a), out.buf!.ptr, BigInt(shapeSize(a.shape)), p0, p1));
    return out;
  }
  neg(a: TensorData): TensorData { return this.unary(Un.NEG, a); }
  exp(a: TensorData): TensorData { return this.unary(Un.EXP, a); }
  log(a: TensorData): TensorData { return this.unary(Un.LOG, a); }
  sqrt(a: TensorData): TensorData { return this.unary(Un.SQRT, a); }
  pow(a: TensorData, e: number): TensorData { return this.unary(Un.POW, a, e); }
  scale(a: TensorData, s: number): TensorData { return this.unary(Un.SCALE, a, s); }
  clamp(a: TensorData, lo: number, hi: number): TensorData { return this.unary(Un.CLAMP, a, lo, hi); }
  gelu(a: TensorData): TensorData { return this.unary(Un.GELU, a); }
  relu(a: TensorData): TensorData { return this.unary(Un.RELU, a); }
  silu(a: TensorData): TensorData { return this.unary(Un.SILU, a); }
  softCap(input: TensorData, cap: number): TensorData { return this.unary(Un.SOFTCAP, input, cap); }

  private unaryBwd(op: number, x: TensorData, g: TensorData, p0 = 0, p1 = 0): TensorData {
    HipBackend.f32(x, g);
    if (shapeSize(x.shape) !== shapeSize(g.shape)) throw new Error("backward: input and gradient sizes differ");
    const out = this.alloc(g.shape);
    check(lib.ah_unary_bwd(op, this.h(x), this.h(g), out.buf!.ptr, BigInt(shapeSize(x.shape)), p0, p1));
    return out;
  }
  geluBackward(input: TensorData, gradOutput: TensorData): TensorData { return this.unaryBwd(UnBwd.GELU, input, gradOutput); }
  reluBackward(input: TensorData, gradOutput: TensorData): TensorData { return this.unaryBwd(UnBwd.RELU, input, gradOutput); }
  siluBackward(input: TensorData, gradOutput: TensorData): TensorData { return this.unaryBwd(UnBwd.SILU, input, gradOutput); }
  clampBackward(input: TensorData, gradOutput: TensorData, lo: number, hi: number): TensorData { return this.unaryBwd(UnBwd.CLAMP, input, gradOutput, lo, hi); }
  softCapBackward(gradOutput: TensorData, input: TensorData, cap: number): TensorData { return this.unaryBwd(UnBwd.SOFTCAP, input, gradOutput, cap); }

  siluMul(a: TensorData, b: TensorData): TensorData {
    HipBackend.f32(a, b);
    const out = this.alloc(a.shape);
    check(lib.ah_silu_mul(this.h(a), this.h(b), out.buf!.ptr, BigInt(shapeSize(a.shape))));
    return out;
  }
  siluMulBackward(a: TensorData, b: TensorData, gradOutput: TensorData): TensorData[] {
    HipBackend.f32(a, b, gradOutput);
    const da = this.alloc(a.shape), db = this.alloc(b.shape);
    check(lib.ah_silu_mul_bwd(this.h(a), this.h(b), this.h(gradOutput), da.buf!.ptr, db.buf!.ptr, BigInt(shapeSize(a.shape))));
    return [da, db];
  }

  residualDropoutAdd(residual: TensorData, projected: TensorData, mask: TensorData): TensorData {
    HipBackend.f32(residual, projected);
    const out = this.alloc(residual.shape);
    check(lib.ah_residual_dropout_add(this.h(residual), this.h(projected), mask ? this.h(mask) : 0n, out.buf!.ptr, BigInt(shapeSize(residual.shape))));
    return out;
  }
  /** Bit-equal to DropoutRng on the CPU (packages/autograd/src/ops.ts:25-82) for every index. */
  dropoutMask(shape: Shape, seed: number, counter: number, p: number): TensorData {
    const out = this.alloc(shape);
    check(lib.ah_dropout_mask(out.buf!.ptr, BigInt(shapeSize(shape)), seed | 0, counter | 0, p));
    return out;
  }
  addInplace(a: TensorData, b: TensorData): void {
    HipBackend.f32(a, b);
    if (shapeSize(a.shape) !== shapeSize(b.shape)) throw new Error("addInplace: size mismatch");
    check(lib.ah_add_inplace(this.h(a), this.h(b), BigInt(shapeSize(a.shape))));
    this.dirty(a);
  }
  scaleInplace(a: TensorData, scalar: number): void {
    HipBackend.f32(a);
    check(lib.ah_scale_inplace(this.h(a), scalar, BigInt(shapeSize(a.shape))));
    this.dirty(a);
  }

  // ── nn ──────────────────────────────────────────────────────────────────
  embedding(weight: TensorData, indices: TensorData): TensorData {
    HipBackend.f32(weight);
    const [vocab, dim] = weight.shape;
    const out = this.alloc([...indices.shape, dim]);
    check(lib.ah_embedding(this.h(weight), this.h(indices), out.buf!.ptr, BigInt(shapeSize(indices.shape)), BigInt(dim), BigInt(vocab), Dt.F32));
    return out;
  }
  embeddingBackward(indices: TensorData, gradOutput: TensorData, vocabSize: number): TensorData {
    HipBackend.f32(gradOutput);
    const dim = gradOutput.shape.at(-1)!;
    const out = this.alloc([vocabSize, dim]);
    check(lib.ah_embedding_bwd(this.h(indices), this.h(gradOutput), out.buf!.ptr, BigInt(shapeSize(indices.shape)), BigInt(dim), BigInt(vocabSize), 0));
    return out;
  }
  layerNorm(x: TensorData, weight: TensorData, bias: TensorData, eps: number): TensorData {
    HipBackend.f32(x, weight, bias);
    const dim = x.shape.at(-1)!;
    if (shapeSize(weight.shape) !== dim || shapeSize(bias.shape) !== dim) throw new Error("layerNorm: weight/bias length must equal the last dimension");
    const out = this.alloc(x.shape);
    check(lib.ah_layernorm(this.h(x), this.h(weight), this.h(bias), out.buf!.ptr, BigInt(shapeSize(x.shape) / Math.max(1, dim)), BigInt(dim), eps, Dt.F32, Dt.F32));
    return out;
  }
  layerNormBackward(x: TensorData, weight: TensorData, gradOutput: TensorData, eps: number): { dx: TensorData; dw: TensorData; db: TensorData } {
    HipBackend.f32(x, weight, gradOutput);
    const dim = x.shape.at(-1)!;
    const dx = this.alloc(x.shape), dw = this.alloc(weight.shape), db = this.alloc(weight.shape);
    check(lib.ah_layernorm_bwd(this.h(x), this.h(weight), this.h(gradOutput), Dt.F32, 0n, dx.buf!.ptr, 0n, dw.buf!.ptr, db.buf!.ptr,
      BigInt(shapeSize(x.shape) / Math.max(1, dim)), BigInt(dim), eps, 0, Dt.F32));
    return { dx, dw, db };
  }
  softmax(a: TensorData, axis?: number): TensorData { return this.softmaxImpl(a, axis, 0); }
  logSoftmax(a: TensorData, axis?: number): TensorData { return this.softmaxImpl(a, axis, 1); }
  private softmaxImpl(a: TensorData, axis: number | undefined, log: number): TensorData {
    HipBackend.f32(a);
    const ax = HipBackend.axis(axis === undefined ? a.shape.length - 1 : axis, a.shape.length);
    const out = this.alloc(a.shape);
    check(lib.ah_softmax(this.h(a), out.buf!.ptr, BigInt(shapeSize(a.shape.slice(0, ax))), BigInt(a.shape[ax]), BigInt(shapeSize(a.shape.slice(ax + 1))), log));
    return out;
  }

  /** The row log-sum-exp of the last crossEntropy on a logits tensor, kept for crossEntropyBackward on the same logits. */
  private ceLse = new WeakMap<TensorData, DeviceTensor>();
  crossEntropy(logits: TensorData, targets: TensorData): TensorData {
    HipBackend.f32(logits);
    const [N, C] = logits.shape;
    const out = this.alloc([]), lse = this.alloc([N]);
    check(lib.ah_cross_entropy(this.h(logits), Dt.F32, this.h(targets), out.buf!.ptr, lse.buf!.ptr, BigInt(N), BigInt(C)));
    this.ceLse.set(logits, lse);
    return out;
  }
  crossEntropyBackward(logits: TensorData, targets: TensorData, gradOutput: TensorData): TensorData {
    HipBackend.f32(logits, gradOutput);
    const [N, C] = logits.shape;
    let lse = this.ceLse.get(logits), own = false;
    if (lse === undefined || lse.buf === null) {
      const tmp = this.alloc([]);
      lse = this.alloc([N]);
      own = true;
      check(lib.ah_cross_entropy(this.h(logits), Dt.F32, this.h(targets), tmp.buf!.ptr, lse.buf!.ptr, BigInt(N), BigInt(C)));
      this.releaseGpuTensor(tmp);
    }
    const out = this.alloc([N, C]);
    check(lib.ah_cross_entropy_bwd(this.h(logits), Dt.F32, this.h(targets), lse.buf!.ptr, this.h(gradOutput), 1.0, out.buf!.ptr, BigInt(N), BigInt(C)));
    if (own) this.releaseGpuTensor(lse);
    return out;
  }

  // ── reshape / slice ─────────────────────────────────────────────────────
  reshape(a: TensorData, shape: Shape): TensorData {
    if (shapeSize(shape) !== shapeSize(a.shape)) throw new Error(`Cannot reshape [${a.shape}] to [${shape}]: size mismatch`);
    return this.view(a, shape);
  }
  transpose(a: TensorData, dim0: number, dim1: number): TensorData {
    const nd = a.shape.length, d0 = HipBackend.axis(dim0, nd), d1 = HipBackend.axis(dim1, nd);
    const ns = [...a.shape];
    ns[d0] = a.shape[d1]; ns[d1] = a.shape[d0];
    HipBackend.words(a);
    const out = this.alloc(ns, a.dtype);
    check(lib.ah_transpose(this.h(a), out.buf!.ptr, nd, addressOf(i64s(a.shape)), d0, d1));
    return out;
  }
  slice(a: TensorData, starts: number[], ends: number[]): TensorData {
    HipBackend.words(a);
    const out = this.alloc(starts.map((s, i) => ends[i] - s), a.dtype);
    check(lib.ah_slice(this.h(a), out.buf!.ptr, a.shape.length, addressOf(i64s(a.shape)), addressOf(i64s(starts)), addressOf(i64s(ends))));
    return out;
  }
  scatterSlice(grad: TensorData, origShape: Shape, starts: number[], _ends: number[]): TensorData {
    HipBackend.words(grad);
    const out = this.alloc(origShape, grad.dtype);
    check(lib.ah_scatter_slice(this.h(grad), out.buf!.ptr, origShape.length, addressOf(i64s(grad.shape)), addressOf(i64s(origShape)), addressOf(i64s(starts))));
    return out;
  }
  sliceQkv(a: TensorData): [TensorData, TensorData, TensorData] {
    const [rows, c3] = a.shape, d = Math.floor(c3 / 3);
    HipBackend.words(a);
    const q = this.alloc([rows, d]), k = this.alloc([rows, d]), v = this.alloc([rows, d]);
    check(lib.ah_slice_qkv(this.h(a), q.buf!.ptr, k.buf!.ptr, v.buf!.ptr, BigInt(rows), BigInt(d)));
    return [q, k, v];
  }
  cat(tensors: TensorData[], axis: number): TensorData {
    if (tensors.length === 0) throw new Error("cat: empty tensor list");
    const nd = tensors[0].shape.length, ax = HipBackend.axis(axis, nd);
    const oshape = [...tensors[0].shape];
    for (const t of tensors.slice(1))
      for (let d = 0; d < nd; d++) {
        if (d === ax) oshape[d] += t.shape[d];
        else if (t.shape[d] !== oshape[d]) throw new Error(`cat: shape mismatch at dim ${d}`);
      }
    HipBackend.words(...tensors);
    const out = this.alloc(oshape, tensors[0].dtype);
    let off = 0;
    for (const t of tensors) {
      check(lib.ah_cat_part(this.h(t), out.buf!.ptr, nd, addressOf(i64s(t.shape)), addressOf(i64s(oshape)), ax, BigInt(off)));
      off += t.shape[ax];
    }
    return out;
  }
  broadcast(a: TensorData, targetShape: Shape): TensorData {
    const nd = targetShape.length;
    const src = [...new Array(nd - a.shape.length).fill(1), ...a.shape];
    HipBackend.words(a);
    const out = this.alloc(targetShape, a.dtype);
    check(lib.ah_broadcast(this.h(a), out.buf!.ptr, nd, addressOf(i64s(targetShape)), addressOf(i64s(HipBackend.bstrides(src, targetShape)))));
    return out;
  }
  castDtype(a: TensorData, dtype: Dtype): TensorData {
    if (dtype === a.dtype) return a;
    const out = this.alloc(a.shape, dtype);
    check(lib.ah_cast(this.h(a), DT_CODE[a.dtype], out.buf!.ptr, DT_CODE[dtype], BigInt(shapeSize(a.shape))));
    return out;
  }

  // ── utility ─────────────────────────────────────────────────────────────
  /** First maximum wins, NaN is never selected (packages/tensor/src/cpu_ref.ts:698-756); the result is i32. */
  argmax(a: TensorData, axis?: number): TensorData {
    HipBackend.f32(a);
    if (axis === undefined) {
      const out = this.alloc([], "i32");
      check(lib.ah_argmax(this.h(a), out.buf!.ptr, 1n, BigInt(shapeSize(a.shape)), 1n));
      return out;
    }
    const ax = HipBackend.axis(axis, a.shape.length);
    const oshape = a.shape.filter((_, i) => i !== ax);
    const out = this.alloc(oshape.length ? oshape : [1], "i32");
    check(lib.ah_argmax(this.h(a), out.buf!.ptr, BigInt(shapeSize(a.shape.slice(0, ax))), BigInt(a.shape[ax]), BigInt(shapeSize(a.shape.slice(ax + 1)))));
    return out;
  }
  /** Sampling-path helper, never called from the training step: host selection over a read-back, in the reference's order
   *  (descending value, earlier index first among equals; packages/tensor/src/cpu_ref.ts:758-819). */
  topk(a: TensorData, k: number, axis?: number): { values: TensorData; indices: TensorData } {
    const nd = a.shape.length, ax = HipBackend.axis(axis === undefined ? nd - 1 : axis, nd);
    const dim = a.shape[ax];
    if (k > dim) throw new Error(`topk: k=${k} exceeds axis size ${dim}`);
    const outer = shapeSize(a.shape.slice(0, ax)), inner = shapeSize(a.shape.slice(ax + 1));
    const src = a.data, vals = new Float32Array(outer * k * inner), idxs = new Int32Array(outer * k * inner);
    const order = new Array<number>(dim);
    for (let o = 0; o < outer; o++)
      for (let i = 0; i < inner; i++) {
        for (let d = 0; d < dim; d++) order[d] = d;
        const at = (d: number) => src[(o * dim + d) * inner + i];
        order.sort((x, y) => (at(y) - at(x)) || (x - y));
        for (let j = 0; j < k; j++) { vals[(o * k + j) * inner + i] = at(order[j]); idxs[(o * k + j) * inner + i] = order[j]; }
      }
    const oshape = a.shape.map((d, i) => (i === ax ? k : d));
    return { values: { shape: oshape, dtype: a.dtype, data: vals }, indices: { shape: oshape, dtype: "i32", data: idxs } };
  }
  /** Not on the training path (packages/tensor/src/cpu_ref.ts:821-845): host gather of a read-back. */
  gather(a: TensorData, axis: number, indices: TensorData): TensorData {
    const ax = HipBackend.axis(axis, a.shape.length);
    const inner = shapeSize(a.shape.slice(ax + 1)), dim = a.shape[ax];
    const iInner = shapeSize(indices.shape.slice(ax + 1)), iDim = indices.shape[ax];
    const src = a.data, ind = indices.data, out = new (dtypeArray(a.dtype))(shapeSize(indices.shape));
    for (let p = 0; p < out.length; p++) {
      const o = Math.floor(p / (iDim * iInner)), i = p % iInner;
      out[p] = src[(o * dim + ind[p]) * inner + i];
    }
    return { shape: [...indices.shape], dtype: a.dtype, data: out };
  }
  clone(a: TensorData): TensorData {
    const out = this.alloc(a.shape, a.dtype);
    check(lib.ah_copy(out.buf!.ptr, this.h(a), BigInt(shapeSize(a.shape) * DT_BYTES[a.dtype])));
    return out;
  }
  equal(a: TensorData, b: TensorData): boolean {
    if (a.dtype !== b.dtype || a.shape.length !== b.shape.length || !a.shape.every((d, i) => d === b.shape[i])) return false;
    const x = a.data, y = b.data;
    for (let i = 0; i < x.length; i++) if (x[i] !== y[i]) return false;
    return true;
  }
  allClose(a: TensorData, b: TensorData, atol = 1e-5, rtol = 1e-8): boolean {
    if (a.shape.length !== b.shape.length || !a.shape.every((d, i) => d === b.shape[i])) return false;
    const x = a.data, y = b.data;
    for (let i = 0; i < x.length; i++) if (Math.abs(x[i] - y[i]) > atol + rtol * Math.abs(y[i])) return false;
    return true;
  }

  // ── mask ────────────────────────────────────────────────────────────────
  causalMask(size: number): TensorData {
    const out = this.alloc([size, size]);
    check(lib.ah_causal_mask(out.buf!.ptr, BigInt(size)));
    return out;
  }
  maskedFill(a: TensorData, mask: TensorData, value: number): TensorData {
    HipBackend.f32(a, mask);
    const out = this.alloc(a.shape);
    check(lib.ah_masked_fill(this.h(a), this.h(mask), out.buf!.ptr, BigInt(shapeSize(a.shape)), BigInt(shapeSize(mask.shape)), value));
    return out;
  }

  // ── flash attention (interfaces.ts:127-135): Q, K, V [B*H, T, D], every slab on its own ─────────────────────
  private flash(Q: TensorData, K: TensorData, V: TensorData, T: number, scale: number, softCap: number): Struct<"AhFlash"> {
    const [BH, T2, D] = Q.shape;
    const same = (x: TensorData) => x.shape.length === 3 && x.shape.every((d, i) => d === Q.shape[i]);
    if (T2 !== T || !same(K) || !same(V)) throw new Error("flashAttention: Q, K, V must all be [B*H, T, D]");
    const f = this.flashDesc;
    f.i32("dtype", Dt.F32).i32("batch", BH).i32("heads", 1).i32("seq", T).i32("head_dim", D);
    for (const p of ["q", "k", "v", "o"]) f.i64(p + "_sb", T * D).i64(p + "_sh", 0).i64(p + "_st", D);
    f.f32("scale", scale).f32("soft_cap", softCap).i32("bwd_variant", 0).i32("reserved", 0);
    return f;
  }
  flashAttention(Q: TensorData, K: TensorData, V: TensorData, T: number, scale: number, softCap: number): { output: TensorData; lse: TensorData } {
    const f = this.flash(Q, K, V, T, scale, softCap);
    const output = this.alloc(Q.shape), lse = this.alloc([Q.shape[0], T]);
    f.u64("q", this.h(Q)).u64("k", this.h(K)).u64("v", this.h(V)).u64("o", output.buf!.ptr).u64("lse", lse.buf!.ptr);
    check(lib.ah_flash_fwd(f.p));
    return { output, lse };
  }
  flashAttentionBackward(Q: TensorData, K: TensorData, V: TensorData, O: TensorData, dO: TensorData, lse: TensorData,
                         T: number, scale: number, softCap: number): { dQ: TensorData; dK: TensorData; dV: TensorData } {
    const f = this.flash(Q, K, V, T, scale, softCap);
    const dQ = this.alloc(Q.shape), dK = this.alloc(Q.shape), dV = this.alloc(Q.shape);
    f.u64("q", this.h(Q)).u64("k", this.h(K)).u64("v", this.h(V)).u64("o", this.h(O)).u64("lse", this.h(lse));
    f.u64("d_o", this.h(dO)).u64("dq", dQ.buf!.ptr).u64("dk", dK.buf!.ptr).u64("dv", dV.buf!.ptr);
    check(lib.ah_flash_bwd(f.p));
    return { dQ, dK, dV };
  }

  // ── reductions / optimizer ──────────────────────────────────────────────
  sumOfSquares(data: TensorData): TensorData {
    HipBackend.f32(data);
    const out = this.alloc([1]);
    check(lib.ah_sum_sq(this.h(data), BigInt(shapeSize(data.shape)), out.buf!.ptr));
    return out;
  }
  /** One scalar for the whole gradient set, one launch (packages/train/src/trainer.ts:1345-1349). */
  totalSumOfSquares(tensors: TensorData[]): TensorData {
    const total = this.alloc([1]);
    HipBackend.f32(...tensors);
    const n = tensors.length, xs = new BigUint64Array(Math.max(n, 1)), ns = new BigUint64Array(Math.max(n, 1));
    tensors.forEach((t, i) => { xs[i] = this.h(t); ns[i] = BigInt(shapeSize(t.shape)); });
    check(lib.ah_sum_sq_list(addressOf(xs), addressOf(ns), n, total.buf!.ptr));
    return total;
  }
  /** 0.0 when every element is finite, 1.0 otherwise (packages/tests/src/gpu-perf.test.ts:106-149). */
  checkFinite(data: TensorData): TensorData {
    HipBackend.f32(data);
    const out = this.alloc([1]);
    check(lib.ah_check_finite(this.h(data), BigInt(shapeSize(data.shape)), out.buf!.ptr));
    return out;
  }
  /** packages/train/src/optimizers.ts:54-94.  The scalars that are the same for every tensor of a step live in a small
   *  device struct written once per step; the by-value argument carries the weight decay only, so a recorded step plan
   *  needs no node rewritten when the learning rate moves. */
  adamwStep(params: TensorData, grads: TensorData, m: TensorData, v: TensorData, lr: number, beta1: number, beta2: number, eps: number,
            weightDecay: number, bc1: number, bc2: number, gradScale = 1.0): void {
    HipBackend.f32(params, grads, m, v);
    const n = shapeSize(params.shape);
    if (n !== shapeSize(grads.shape) || n !== shapeSize(m.shape) || n !== shapeSize(v.shape)) throw new Error("adamwStep: params, grads, m, v must have the same size");
    const key = [lr, beta1, beta2, eps, bc1, bc2, gradScale].join(",");
    this.hyper ??= new Buf(32);
    const a = this.adamDesc;
    if (key !== this.hyperKey) {
      a.f32("lr", lr).f32("beta1", beta1).f32("beta2", beta2).f32("eps", eps).f32("weight_decay", 0).f32("bc1", bc1).f32("bc2", bc2).f32("grad_scale", gradScale);
      check(lib.ah_upload(this.hyper.ptr, a.p, 32n));
      this.hyperKey = key;
    }
    a.f32("lr", 0).f32("beta1", 0).f32("beta2", 0).f32("eps", 0).f32("weight_decay", weightDecay).f32("bc1", 0).f32("bc2", 0).f32("grad_scale", 0);
    check(lib.ah_adamw(this.h(params), this.h(grads), this.h(m), this.h(v), BigInt(n), a.p, this.hyper.ptr, 0n, 0n));
    this.dirty(params); this.dirty(m); this.dirty(v);
  }
}
