"""Benchmark of the DiT attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload wan14b|wan14b-ring|wan14b-ulysses|wan14b-usp|wan14b-fp8|wan1.3b|flux-dev]

One step = one pass of the path over one synthetic batch already resident in HBM: fused q/k
RMSNorm + RoPE, then the bf16 self-attention forward (with LSE).  Prints ONE JSON line:
`value` is attention TFLOP/s over the whole step (4*B*H*Sq*Skv*D FLOP / step time); `roofline`
is the attention kernel alone, timed with events on the launch stream; `roofline_norm_rope` is the
prologue kernel against HBM peak; `cpu_baseline` is the oracle's restatement of the reference's
`dot_product` path timed on the host cores over a bounded slice of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_FP8_TFLOPS = 5000.0  # MI355X dense fp8 MFMA
PEAK_HBM_GBPS = 8000.0  # MI355X HBM3E


def cpu_baseline(workload, budget_rows: int):
  """The oracle's bf16-flow `dot_product` (attention_flax.py:1487-1567 restated in numpy), one head,
  one block of query rows against every key of the workload, on the host cores."""
  import numpy as np

  import oracle as O

  rows = min(budget_rows, workload.seq)
  block = 2048  # query rows per call: bounds the [rows, keys] score matrix to ~0.6 GB in f32
  q = O.normal_bf16((1, rows, 128), 0)
  k = O.normal_bf16((1, workload.kv_seq, 128), 1)
  v = O.normal_bf16((1, workload.kv_seq, 128), 2)
  O.attention_dot_product_bf16(q[:, :64], k[:, :1024], v[:, :1024], workload.scale)  # first call untimed
  t0 = time.perf_counter()
  for r0 in range(0, rows, block):
    O.attention_dot_product_bf16(q[:, r0:r0 + block], k, v, workload.scale)
  dt = time.perf_counter() - t0
  flops = O.attention_flops(1, 1, rows, workload.kv_seq, 128)
  cores = int(os.environ.get("OMP_NUM_THREADS", 0)) or os.cpu_count()
  return {
      "value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
      "sample": f"1 head x {rows} query rows x {workload.kv_seq} keys (of {workload.heads} heads x {workload.seq} rows), "
                f"numpy restatement of dot_product with bf16 score/prob rounding, {dt:.2f} s; not JAX (absent from the image)",
  }


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=10)
  ap.add_argument("--warmup", type=int, default=3)
  ap.add_argument("--workload", default=None,
                  help="default wan14b; a run without this option also reports the backward blocks of --with-backward "
                       "(a failure there is reported in the block and does not cost the headline line)")
  ap.add_argument("--cpu-rows", type=int, default=16384, help="query rows of the CPU-baseline slice (0: skip)")
  ap.add_argument("--traffic-probe", action="store_true",
                  help="also launch one 1 GiB device copy: the plain copy kernel of known size that scales rocprofv3's "
                       "FETCH_SIZE / WRITE_SIZE counters")
  ap.add_argument("--separate-merge", action="store_true",
                  help="ring workloads: one attention launch and one merge launch per KV chunk instead of the fused step")
  ap.add_argument("--fused-qkv", action="store_true",
                  help="also time the prologue over a fused q|k|v projection output [1,S,3*H*D] with the three Linear biases "
                       "(mdattn_norm_rope_qkv, in place), outside the timed steps; reported as `roofline_norm_rope_qkv`")
  ap.add_argument("--key-split", type=int, default=0, metavar="F",
                  help="also time the self-attention with its key range split F ways inside ONE launch (the splits ride as batch "
                       "entries: q with batch stride 0, k / v viewed [F, Skv/F, H, D]), followed by F merges and the finalize; "
                       "reported as `key_split` beside the headline.  Skv must be divisible by F")
  ap.add_argument("--hbm-probe", action="store_true",
                  help="also time the runtime's own streaming kernels on tensors of the prologue's size (copy, two-input add, "
                       "fill, sum): what this machine's memory system gives plain kernels, for scale; reported as `hbm_probe`")
  ap.add_argument("--mfma-probe", action="store_true",
                  help="also run the library's MFMA rate probe: MFMA 32x32x16 bf16 back to back on the workload's kind of "
                       "operands (N(0,1) rounded to bf16) and on zeros, alone and with the LDS reads / softmax instructions of "
                       "an attention loop beside them; reported as `mfma_probe` (what this machine sustains, against the "
                       "published peak)")
  ap.add_argument("--atomic-probe", action="store_true",
                  help="with --with-backward: also time the f32 atomic adds that a single-pass backward (five matrix products "
                       "instead of seven) would issue for dq at this shape, per wave and reduced per workgroup; reported inside "
                       "the `backward` object")
  ap.add_argument("--with-mask", action="store_true",
                  help="fp8 workloads: also time the attention with a key padding mask (1000 keys excluded), beside the "
                       "unmasked call with the same softmax, for power-of-two and for arbitrary scales; reported inside `roofline_exp2`")
  ap.add_argument("--with-backward", action="store_true",
                  help="also time the backward pass (dq, dk, dv) of the workload's attention, outside the timed steps; "
                       "reported as a `backward` object beside the headline")
  args = ap.parse_args()
  default_run = args.workload is None  # the plain `python bench.py [--gpus 1 --steps K --warmup W]` form
  args.workload = args.workload or "wan14b"
  explicit_backward = args.with_backward
  args.with_backward = args.with_backward or default_run
  if args.gpus != 1:
    print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
    sys.exit(2)

  import torch

  import oracle as O
  from maxdiffusion_amd import _lib, ops
  from maxdiffusion_amd.build import ensure_built

  ensure_built()
  _lib.load()
  if not torch.cuda.is_available():
    raise RuntimeError("bench.py needs a GPU: the hot path has no CPU implementation")
  dev = torch.device("cuda:0")
  w = O.WORKLOADS[args.workload]
  H, D, S, Skv = w.heads, w.head_dim, w.seq, w.kv_seq
  ring = max(w.ring_chunks, 1)

  gen = torch.Generator(device=dev).manual_seed(0)
  randn = lambda *shape: torch.randn(shape, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
  tb = lambda x: torch.from_numpy(O.to_bf16_bits(x).view("int16")).view(torch.bfloat16).to(dev)
  # pre-norm projections q, k [1,S,H*D] and v, N(0,1) in bf16; norm weights 1 + 0.1 N(0,1)
  q_in, k_in = randn(1, S, H * D), randn(1, S, H * D)
  v = randn(1, Skv * ring, H, D)
  k_extra = randn(1, Skv * (ring - 1), H, D) if ring > 1 else None
  fp8 = args.workload.endswith("-fp8")
  # bf16: the prologue emits q * scale * log2(e) (still one rounding) and the attention kernel is given scale = ln 2,
  # so that it sees scale * log2(e) == 1 and its logits need no multiply; same result as scale = D^-1/2 on plain q
  q_mul = 1.0 if fp8 else ops.folded_q_mul(D, w.scale)
  att_scale = w.scale if fp8 else ops.FOLDED_SCALE
  if w.norm == "fullrow":
    wq, wk = tb(O.norm_weight(H * D, 3)), tb(O.norm_weight(H * D, 4))
    # a ring shard owns the first S tokens of the full latent grid
    cos, sin = (torch.from_numpy(t[:S].copy()).to(dev) for t in O.wan_rope_table(w.grid, D))
    prologue = lambda: ops.norm_rope_fullrow(q_in, k_in, wq, wk, cos, sin, H, q_mul=q_mul)
  elif w.norm == "rows":  # LTX-2: f32 weights, cos / sin of the size of the tensor (interleaved form), one call per tensor
    wq, wk = (torch.from_numpy(O.norm_weight(H * D, s_)).to(dev) for s_ in (3, 4))
    ang = torch.rand((1, S, H * D), generator=gen, device=dev, dtype=torch.float32) * 6.2831853
    cos, sin = torch.cos(ang), torch.sin(ang)
    del ang
    prologue = lambda: (ops.norm_rope_rows(q_in, wq * q_mul, cos, sin, heads=H, mode="interleaved"),
                        ops.norm_rope_rows(k_in, wk, cos, sin, heads=H, mode="interleaved"))
  else:
    wq, wk = tb(O.norm_weight(D, 3)), tb(O.norm_weight(D, 4))
    cos, sin = (torch.from_numpy(t).to(dev) for t in O.flux_rope_table(O.flux_ids(*w.grid)))
    q4, k4 = q_in.view(1, S, H, D), k_in.view(1, S, H, D)
    prologue = lambda: ops.norm_rope_perhead(q4, k4, wq, wk, cos, sin, q_mul=q_mul)

  ev = lambda: torch.cuda.Event(enable_timing=True)
  t_pro, t_att, t_quant = [], [], []

  def step(record: bool):
    e0, e1, e2, eq = ev(), ev(), ev(), ev()
    e0.record()
    qn, kn = prologue()
    e1.record()
    if fp8:  # per-tensor absmax e4m3 quantisation of q, k, v, then the fp8 kernel
      # q's quantiser carries scale * log2(e); power-of-two q and k scales: the kernel scales the logits in its MFMAs
      q8, sq = ops.quant_e4m3(qn, premul=ops.folded_q_mul(D, w.scale), pow2_scale=True)
      k8, sk = ops.quant_e4m3(kn, pow2_scale=True)
      v8, sv = ops.quant_e4m3(v)
      eq.record()
      # the softmax mode the registry entry hip_flash_fp8 asks for; the exact-exponential mode is timed below
      ops.flash_attention_fp8(q8, k8, v8, sq, sk, sv, scale=ops.FOLDED_SCALE, return_lse=True, softmax="byte_grid")
    elif ring == 1:
      ops.flash_attention(qn, kn, v, scale=att_scale, return_lse=True)
    else:  # one ring shard: this Q chunk against `ring` successive KV chunks, merged in LSE space
      o_run, l_run = ops.new_merge_state(1, S, H, D, dev)
      for i in range(ring):
        kc = kn if i == 0 else k_extra[:, (i - 1) * Skv:i * Skv]
        if args.separate_merge:
          o, l = ops.flash_attention(qn, kc, v[:, i * Skv:(i + 1) * Skv], scale=att_scale, return_lse=True)
          ops.merge_partial(o_run, l_run, o, l)
        else:  # attention and merge in one launch
          ops.flash_attention_merge(qn, kc, v[:, i * Skv:(i + 1) * Skv], o_run, l_run, scale=att_scale)
      ops.finalize(o_run)
    e2.record()
    if record:
      torch.cuda.synchronize()
      t_pro.append(e0.elapsed_time(e1))
      t_att.append((eq if fp8 else e1).elapsed_time(e2))
      if fp8:
        t_quant.append(e1.elapsed_time(eq))

  if args.traffic_probe:
    src = torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)
    dst = torch.empty_like(src)
    dst.copy_(src)  # reads 1 GiB, writes 1 GiB
    torch.cuda.synchronize()
    del src, dst
  for _ in range(args.warmup):
    step(False)
  torch.cuda.synchronize()
  t0 = time.perf_counter()
  for _ in range(args.steps):
    step(True)
  torch.cuda.synchronize()
  ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

  # the prologue kernel runs for ~0.55 ms: an event pair around a single launch also sees the launch gap, so its
  # roofline figure comes from 20 launches issued back to back between one event pair (outside the timed steps)
  reps = 20
  e0, e1 = ev(), ev()
  e0.record()
  for _ in range(reps):
    prologue()
  e1.record()
  torch.cuda.synchronize()
  pro_ms = e0.elapsed_time(e1) / reps

  # the prologue over one fused q|k|v projection output, biases folded in, written back in place
  fused_qkv = None
  if args.fused_qkv and w.norm == "fullrow":
    qkv = randn(1, S, 3 * H * D)
    b3 = (randn(3 * H * D).float() * 0.5).to(torch.bfloat16)
    run = lambda: ops.norm_rope_qkv(qkv, wq, wk, cos, sin, H, bias=b3, q_mul=q_mul, inplace=True)
    run()
    e0, e1 = ev(), ev()
    e0.record()
    for _ in range(reps):
      run()
    e1.record()
    torch.cuda.synchronize()
    fms = e0.elapsed_time(e1) / reps
    fbytes = 2 * 3 * S * H * D * 2 + 2 * S * (D // 2) * 4 + 2 * 2 * H * D * 2 + 3 * H * D * 2  # q, k, v read and written; tables; weights; bias
    fused_qkv = {"bound": "hbm", "achieved": fbytes / (fms * 1e-3) / 1e9, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                 "frac": fbytes / (fms * 1e-3) / 1e9 / PEAK_HBM_GBPS, "traffic": None,
                 "kernel": "norm_rope_fullrow_kernel<., true> (fused q|k|v projection, biases added, in place)",
                 "kernel_ms": fms, "bytes_per_launch": fbytes}
    del qkv

  # fp8: the same attention with exact exponentials (mdattn_fwd_fp8's other softmax mode: the lse is then the exact
  # logsumexp of the quantised logits), outside the timed steps
  fp8_exp2 = None
  if fp8:
    qn, kn = prologue()
    q8, sq = ops.quant_e4m3(qn, premul=ops.folded_q_mul(D, w.scale), pow2_scale=True)
    k8, sk = ops.quant_e4m3(kn, pow2_scale=True)
    v8, sv = ops.quant_e4m3(v)
    run = lambda: ops.flash_attention_fp8(q8, k8, v8, sq, sk, sv, scale=ops.FOLDED_SCALE, return_lse=True, softmax="exp2")
    run()
    e0, e1 = ev(), ev()
    e0.record()
    for _ in range(5):
      run()
    e1.record()
    torch.cuda.synchronize()
    ems = e0.elapsed_time(e1) / 5
    efl = O.attention_flops(1, H, S, Skv, D)
    fp8_exp2 = {"bound": "mfma", "achieved": efl / (ems * 1e-3) / 1e12, "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                "frac": efl / (ems * 1e-3) / 1e12 / PEAK_FP8_TFLOPS, "traffic": None, "kernel": "attn_fwd_fp8_kernel<4,1> (softmax_mode exp2)",
                "kernel_ms": ems, "flop_per_launch": efl}
    if args.with_mask:
      # the same call with a key padding mask (the last 1000 keys excluded), with power-of-two scales and with
      # arbitrary ones, each beside its unmasked twin
      keep = torch.ones((1, Skv), dtype=torch.bool, device=dev)
      keep[:, Skv - 1000:] = False
      kb = ops.key_mask_bias(keep)

      def t5(fn):
        fn()
        e0, e1 = ev(), ev()
        e0.record()
        for _ in range(5):
          fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / 5

      fp8_exp2["masked"] = {
          "masked_keys": 1000, "unmasked_ms": ems,
          "masked_ms": t5(lambda: ops.flash_attention_fp8(q8, k8, v8, sq, sk, sv, scale=ops.FOLDED_SCALE, key_bias=kb)),
          "unmasked_arbitrary_scale_ms": t5(lambda: ops.flash_attention_fp8(q8, k8, v8, sq, sk, sv, scale=0.1)),
          "masked_arbitrary_scale_ms": t5(lambda: ops.flash_attention_fp8(q8, k8, v8, sq, sk, sv, scale=0.1, key_bias=kb))}
    del q8, k8, v8

  # configs[2] also names the cross-attention of the same Q against 512 text tokens (no RoPE): reported beside the
  # headline figure, outside the timed steps
  cross = None
  if w.cross_kv and not fp8:
    qn, _ = prologue()
    kc, vc = randn(1, w.cross_kv, H, D), randn(1, w.cross_kv, H, D)
    for _ in range(2):
      ops.flash_attention(qn, kc, vc, scale=att_scale, return_lse=True)
    e0, e1 = ev(), ev()
    e0.record()
    for _ in range(reps):
      ops.flash_attention(qn, kc, vc, scale=att_scale, return_lse=True)
    e1.record()
    torch.cuda.synchronize()
    cms = e0.elapsed_time(e1) / reps
    cfl = O.attention_flops(1, H, S, w.cross_kv, D)
    cross = {"Skv": w.cross_kv, "kernel_ms": cms, "TFLOP/s": cfl / (cms * 1e-3) / 1e12,
             "GB/s": (2 * S * H * D * 2 + 2 * w.cross_kv * H * D * 2 + H * S * 4) / (cms * 1e-3) / 1e9}

  # backward of one attention call of the workload (one KV chunk for the ring shards), on the operands the training path
  # hands it: q from the prologue with scale * log2(e) folded in (the configuration of the headline forward), and, for
  # comparison, on plain q with the softmax scale as an argument
  backward = None
  if args.with_backward and not fp8:

    def measure_backward():
      if D not in (64, 128):
        raise SystemExit("--with-backward: the backward kernels are built for head dims 64 and 128")
      vb = v[:, :Skv]
      dout = randn(1, S, H, D)

      def time_backward(qb, kb, sc):
        ob, lb = ops.flash_attention(qb, kb, vb, scale=sc, return_lse=True)
        for _ in range(2):
          ops.flash_attention_backward(qb, kb, vb, ob, dout, lb, scale=sc)
        e0, e1 = ev(), ev()
        e0.record()
        for _ in range(5):
          ops.flash_attention_backward(qb, kb, vb, ob, dout, lb, scale=sc)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / 5, (qb, kb, ob, lb)

      qf, kf = prologue()
      bms, (qb, kb, ob, lb) = time_backward(qf, kf[:, :Skv] if kf.shape[1] != Skv else kf, att_scale)
      if w.norm == "fullrow":
        qp, kp = ops.norm_rope_fullrow(q_in, k_in, wq, wk, cos, sin, H)
      elif w.norm == "rows":
        qp, kp = ops.norm_rope_rows(q_in, wq, cos, sin, heads=H, mode="interleaved"), ops.norm_rope_rows(k_in, wk, cos, sin, heads=H, mode="interleaved")
      else:
        qp, kp = ops.norm_rope_perhead(q4, k4, wq, wk, cos, sin)
      bms_plain, _ = time_backward(qp, kp, w.scale)
      del qp, kp
      # the five matrix products of the backward pass: S, dP, dV, dK, dQ (the two passes execute seven: S and dP are formed in both)
      bfl = 2.5 * O.attention_flops(1, H, S, Skv, D)
      btf = bfl / (bms * 1e-3) / 1e12
      probe = None
      if args.atomic_probe:
        import ctypes

        fn = _lib.load().mdattn_probe_dq_atomics
        fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int] * 5
        fn.restype = ctypes.c_int
        dqf = torch.zeros((H, S // 32 * 32, D), dtype=torch.float32, device=dev)
        probe = {}
        for per_wave, key in ((1, "per_wave_ms"), (0, "per_workgroup_ms")):
          run = lambda: _lib.check(fn(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream), ctypes.c_void_p(dqf.data_ptr()), H, S, Skv, D, per_wave), "probe")
          run()
          e0, e1 = ev(), ev()
          e0.record()
          for _ in range(3):
            run()
          e1.record()
          torch.cuda.synchronize()
          probe[key] = e0.elapsed_time(e1) / 3
        n_add = H * (Skv // 256) * (S // 32) * 32 * D  # per workgroup and query tile: one 32 x D partial
        probe.update({"atomic_adds_per_workgroup_mode": n_add, "atomic_adds_per_wave_mode": 8 * n_add,
                      "note": "f32 atomic adds of the dq partials of a key-outer single pass, nothing else in the launch"})
        del dqf
      backward = {"Sq": S, "Skv": Skv, "ms": bms, "TFLOP/s": btf, "bound": "mfma", "peak": 2500.0, "frac": btf / 2500.0,
                  "frac_executed": btf * 7.0 / 5.0 / 2500.0,
                  "flop_counted": bfl, "ms_plain_scale": bms_plain,
                  "note": "5 matrix products counted, 7 executed (two atomic-free passes: dq; dk and dv); ms: q carries scale * log2(e) "
                          "from the prologue, as in the headline forward; ms_plain_scale: plain q, softmax scale as an argument"}
      if probe:
        backward["single_pass_dq_atomics_probe"] = probe
      return backward

    if default_run and not explicit_backward:
      try:
        backward = measure_backward()
      except Exception as e:  # the optional block must not cost the headline line
        backward = {"error": f"{type(e).__name__}: {e}"}
    else:
      backward = measure_backward()

  # the key range split F ways inside one launch, then merged: what a key split could buy small grids
  key_split = None
  if args.key_split > 1 and not fp8 and ring == 1:
    F = args.key_split
    if Skv % F:
      raise SystemExit(f"--key-split: Skv={Skv} is not divisible by {F}")
    qn, kn = prologue()
    one = lambda: ops.flash_attention(qn, kn, v, scale=att_scale, return_lse=True)
    qv, kv, vv = qn.expand(F, S, H, D), kn.reshape(F, Skv // F, H, D), v.reshape(F, Skv // F, H, D)

    def split_attention():
      return ops.flash_attention(qv, kv, vv, scale=att_scale, return_lse=True)

    def split_step():
      o, l = split_attention()
      o_run, l_run = ops.new_merge_state(1, S, H, D, dev)
      for i in range(F):
        ops.merge_partial(o_run, l_run, o[i:i + 1], l[i:i + 1])
      return ops.finalize(o_run)

    def timed(fn, n=reps):
      for _ in range(2):
        fn()
      e0, e1 = ev(), ev()
      e0.record()
      for _ in range(n):
        fn()
      e1.record()
      torch.cuda.synchronize()
      return e0.elapsed_time(e1) / n

    ks_one, ks_att, ks_all = timed(one), timed(split_attention), timed(split_step)
    err = float((split_step().float() - one()[0].float()).abs().max())
    key_split = {"splits": F, "one_launch_ms": ks_one, "split_attention_launch_ms": ks_att, "split_with_merges_and_finalize_ms": ks_all,
                 "max_abs_diff_vs_one_launch": err}

  hbm_probe = None
  if args.hbm_probe:
    n = S * H * D * 2  # elements of q and k together
    a_, b_ = torch.randn(n, device=dev).to(torch.bfloat16), torch.randn(n, device=dev).to(torch.bfloat16)
    c_ = torch.empty_like(a_)

    def rate(fn, nbytes):
      for _ in range(3):
        fn()
      e0, e1 = ev(), ev()
      e0.record()
      for _ in range(reps):
        fn()
      e1.record()
      torch.cuda.synchronize()
      return nbytes / (e0.elapsed_time(e1) / reps * 1e-3) / 1e9

    hbm_probe = {"unit": "GB/s", "bytes_per_tensor": n * 2,
                 "copy_1r_1w": rate(lambda: c_.copy_(a_), 2 * n * 2), "add_2r_1w": rate(lambda: torch.add(a_, b_, out=c_), 3 * n * 2),
                 "fill_1w": rate(lambda: c_.zero_(), n * 2), "sum_1r": rate(lambda: a_.sum(), n * 2),
                 "note": "torch's own elementwise / reduction kernels on bf16 tensors of the prologue's size"}
    del a_, b_, c_

  # the plain run carries three rows of the probe (registers, the attention loop's mix, zeros): what this machine
  # sustains stands beside the headline in the same line
  mfma_probe = None
  if args.mfma_probe or default_run:

    def measure_mfma_probe():
      import ctypes

      fn = _lib.load().mdattn_probe_mfma_rate
      fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
      fn.restype = ctypes.c_int
      p_iters, p_grid = 20000, 4096  # 2 workgroups of 4 waves per CU at a time, 8 rounds: about 50 ms per launch
      src = torch.randn(32768, device=dev).to(torch.bfloat16)  # 16384 words
      src8 = torch.randn(65536, device=dev).to(torch.float8_e4m3fn)  # 16384 words of e4m3 N(0,1)
      sink = torch.empty(p_grid * 256, dtype=torch.float32, device=dev)
      rows = []
      for mode, what in ((m, t) for m, t in ((0, "MFMA only, operands in registers"), (1, "A operand from LDS for every MFMA"),
                         (2, "A operand from LDS for every second MFMA"),
                         (16, "registers; 1 exp2, 1 add, 1/2 pack per MFMA (head dim 128's softmax)"),
                         (17, "LDS every MFMA; head dim 128's softmax"), (18, "LDS every second MFMA; head dim 128's softmax"),
                         (4, "registers; 2 exp2, 2 add, 1 pack per MFMA (head dim 64's softmax)"),
                         (5, "LDS every MFMA; head dim 64's softmax"), (6, "LDS every second MFMA; head dim 64's softmax"),
                         (8, "MFMA only, all operands zero"), (9, "LDS every MFMA, all operands zero"),
                         (32, "fp8 MFMA 32x32x64 only, operands in registers"), (33, "fp8: A operand (2 KB) from LDS for every MFMA"),
                         (36, "fp8, registers; 4 exp2, 4 add, 2 fp8 packs per MFMA (head dim 128's softmax)"),
                         (37, "fp8, LDS every MFMA; head dim 128's softmax"), (40, "fp8 MFMA only, all operands zero"))
                         if args.mfma_probe or m in (0, 17, 8)):
        is8 = mode >= 32
        p_it = p_iters // 2 if is8 else p_iters  # an fp8 MFMA occupies the pipe for twice the clocks
        run = lambda: _lib.check(fn(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream), mode, p_it, p_grid,
                                    ctypes.c_void_p((src8 if is8 else src).data_ptr()), ctypes.c_void_p(sink.data_ptr())), "mfma probe")
        for _ in range(2):
          run()
        e0, e1 = ev(), ev()
        e0.record()
        for _ in range(3):
          run()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / 3
        # 32 x 32 x 16 x 2 FLOP per bf16 MFMA and wave, four times that per fp8 MFMA
        tf = p_grid * 4 * p_it * 8 * 32768 * (4 if is8 else 1) / (ms * 1e-3) / 1e12
        peak = 5000.0 if is8 else 2500.0
        rows.append({"mode": mode, "what": what, "ms": ms, "TFLOP/s": tf, "peak": peak, "frac_of_peak": tf / peak,
                     "GHz_of_a_full_pipe": tf / peak * 2.4})
      return {"unit": "TFLOP/s", "rows": rows,
              "note": "MFMAs back to back, 2 waves per SIMD, 4 accumulators per wave; the published peaks are 1024 SIMDs x "
                      "one MFMA per 32 clocks (bf16 32x32x16) or 64 clocks (fp8 32x32x64) x 2.4 GHz"}

    if args.mfma_probe:
      mfma_probe = measure_mfma_probe()
    else:
      try:
        mfma_probe = measure_mfma_probe()
      except Exception as e:  # the optional block must not cost the headline line
        mfma_probe = {"error": f"{type(e).__name__}: {e}"}

  # backward of the prologue (input and weight gradients from the saved inputs and the gradients of its outputs)
  prologue_backward = None
  if args.with_backward:

    def measure_prologue_backward():
      gq, gk = randn(1, S, H, D), randn(1, S, H, D)
      if w.norm == "fullrow":
        runb = lambda: ops.norm_rope_fullrow_backward(q_in, k_in, wq, wk, cos, sin, H, gq, gk, q_mul=q_mul)
        nlaunch, pb_bytes = 1, 6 * S * H * D * 2 + 2 * S * (D // 2) * 4 + 2 * H * D * (2 + 4)
        kname_b = "norm_rope_fullrow_bwd_kernel"
      elif w.norm == "rows":
        runb = lambda: (ops.norm_rope_rows_backward(q_in, wq, gq, cos, sin, heads=H, mode="interleaved"),
                        ops.norm_rope_rows_backward(k_in, wk, gk, cos, sin, heads=H, mode="interleaved"))
        nlaunch, pb_bytes = 2, 6 * S * H * D * 2 + 2 * 2 * S * H * D * 4 + 2 * H * D * (4 + 4)
        kname_b = "norm_rope_rows_bwd_kernel (two launches: q, k)"
      else:
        runb = lambda: ops.norm_rope_perhead_backward(q4, k4, wq, wk, cos, sin, gq, gk, q_mul=q_mul)
        nlaunch, pb_bytes = 1, 6 * S * H * D * 2 + 2 * S * (D // 2) * 4 + 2 * D * (2 + 4)
        kname_b = "norm_rope_perhead_bwd_kernel"
      for _ in range(2):
        runb()
      e0, e1 = ev(), ev()
      e0.record()
      for _ in range(reps):
        runb()
      e1.record()
      torch.cuda.synchronize()
      pbms = e0.elapsed_time(e1) / reps
      prologue_backward = {"bound": "hbm", "achieved": pb_bytes / (pbms * 1e-3) / 1e9, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                           "frac": pb_bytes / (pbms * 1e-3) / 1e9 / PEAK_HBM_GBPS, "traffic": None, "kernel": kname_b,
                           "ms": pbms, "bytes_per_call": pb_bytes,
                           "note": "saved inputs and output gradients read once, input gradients written once (bf16), tables, weights and "
                                   "f32 weight gradients; the time includes the second-stage column sum and the workspace allocation"}
      return prologue_backward

    if default_run and not explicit_backward:
      try:
        prologue_backward = measure_prologue_backward()
      except Exception as e:  # the optional block must not cost the headline line
        prologue_backward = {"error": f"{type(e).__name__}: {e}"}
    else:
      prologue_backward = measure_prologue_backward()

  flops = O.attention_flops(1, H, S, Skv * ring, D)
  att_ms = sum(t_att) / len(t_att)
  nr_bytes = O.normrope_bytes(1, S, H, D, with_table=True, per_element_table=w.norm == "rows")
  achieved = flops / (att_ms * 1e-3) / 1e12
  traffic = {}
  tpath = os.path.join(ROOT, "profiles", "traffic.json")
  if os.path.exists(tpath):  # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command
    traffic = json.load(open(tpath)).get(args.workload, {})
  peak = PEAK_FP8_TFLOPS if fp8 else PEAK_BF16_TFLOPS
  kname = "attn_fwd_fp8_kernel" if fp8 else "attn_fwd_bf16_kernel"
  klabel = "attn_fwd_fp8_kernel<4,2> (softmax_mode byte_grid)" if fp8 else kname
  out = {
      "metric": "self-attn TFLOP/s (% bf16 MFMA peak) at Wan-14B 75.6k tokens; norm-RoPE GB/s" if args.workload == "wan14b"
      else f"self-attn TFLOP/s ({args.workload}); norm-RoPE GB/s",
      "value": flops / (ms_per_step * 1e-3) / 1e12,
      "unit": "TFLOP/s",
      "n_gpus": 1,
      "steps": args.steps,
      "warmup": args.warmup,
      "ms_per_step": ms_per_step,
      "higher_is_better": True,
      "scaling": "weak",
      "vs_baseline": None,
      "dtype": "fp8-e4m3" if fp8 else "bf16",
      "data": "synthetic",
      "config": {"workload": f"{args.workload}: B=1 H={H} D={D} Sq={S} Skv={Skv * ring} norm={w.norm} rope={w.rope}"
                             + (f" ring_chunks={ring} ({'attention and merge launched separately' if args.separate_merge else 'merged in the attention launch'})" if ring > 1 else ""),
                 "step": "fused q/k RMSNorm+RoPE -> " + ("per-tensor e4m3 quantisation of q, k, v -> fp8 flash-attention forward with LSE"
                                                             if fp8 else "bf16 flash-attention forward with LSE (softmax scale * log2 e carried by the prologue's q output)")},
      "roofline": {"bound": "mfma", "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
                   "frac": achieved / peak, "traffic": traffic.get(kname), "kernel": klabel,
                   "kernel_ms": att_ms, "flop_per_launch": flops / ring,
                   # spread over the timed steps: the shader clock under this kernel differs from box to box and drifts
                   # within a run, so one average does not place the run; min / median / max do
                   "kernel_ms_min": min(t_att), "kernel_ms_median": sorted(t_att)[len(t_att) // 2], "kernel_ms_max": max(t_att)},
      "roofline_norm_rope": {"bound": "hbm", "achieved": nr_bytes / (pro_ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                             "frac": nr_bytes / (pro_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, "traffic": traffic.get(f"norm_rope_{w.norm}_kernel"),
                             "kernel": f"norm_rope_{w.norm}_kernel" + (" (two launches: q, k)" if w.norm == "rows" else ""),
                             "kernel_ms": pro_ms, "bytes_per_launch": nr_bytes,
                             "in_step_ms": sum(t_pro) / len(t_pro)},
  }
  if fp8:
    out["quant_ms"] = sum(t_quant) / len(t_quant)
    out["roofline_exp2"] = fp8_exp2
  if fused_qkv:
    out["roofline_norm_rope_qkv"] = fused_qkv
  if cross:
    out["cross_attention"] = cross
  if backward:
    out["backward"] = backward
  if prologue_backward:
    out["prologue_backward"] = prologue_backward
  if key_split:
    out["key_split"] = key_split
  if hbm_probe:
    out["hbm_probe"] = hbm_probe
  if mfma_probe:
    out["mfma_probe"] = mfma_probe
  if args.cpu_rows > 0:
    out["cpu_baseline"] = cpu_baseline(w, args.cpu_rows)
  print(json.dumps(out), flush=True)


if __name__ == "__main__":
  main()
