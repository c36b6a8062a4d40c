"""Benchmark: forward pass of the top-2 Mixture-of-Experts layer on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 1..5]

A step is one forward pass of the layer (router -> top-2 gating -> dispatch ->
expert FFN -> combine) over one batch of synthetic tokens that is already
resident in HBM, run through the mtf-shaped API on HipMeshImpl.  Prints ONE
JSON line: whole-job tokens/s, the roofline of the dominant kernel (the expert
grouped GEMM, against the bf16 dense MFMA peak), per-stage timings, and the CPU
restatement of the reference lowering timed on a bounded sample of the same
workload on this machine's host cores.
"""

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)

# Bytes crossing the L2 <-> fabric boundary per grouped-GEMM launch, from
# `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` runs of this script
# (scaled by what the same counters read for a 1 GiB copy: 2.0 and 1.0; the
# summary with the commands is profiles/hbm_traffic_cfg4_pmc.txt).  Mean of the
# wi and wo launches.  Measured offline: the counters cannot be read from here.
MEASURED_GEMM_TRAFFIC_BYTES = {4: 34.0e9}

# MI355X published peaks
HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}

# The five workloads of the benchmark definition.  `cf2` is
# moe_capacity_factor_second_level (hierarchical layer only).
CONFIGS = {
    1: dict(name="cfg1 v1 fp32 2048 tok, d_model 512, d_ff 2048, 8 experts",
            layer="v1", dtype="f32", batch=2, length=1024, group=1024, M=512,
            H=2048, E=8, cf=1.25),
    2: dict(name="cfg2 v1 bf16 16384 tok, d_model 1024, d_ff 4096, 32 experts",
            layer="v1", dtype="bf16", batch=16, length=1024, group=1024,
            M=1024, H=4096, E=32, cf=1.25),
    3: dict(name="cfg3 v1 bf16 skewed 32768 tok, d_model 1024, d_ff 4096, "
                 "64 experts, Zipf(1.2) router bias scaled to 3.0",
            layer="v1", dtype="bf16", batch=16, length=2048, group=2048,
            M=1024, H=4096, E=64, cf=1.0, skew=True),
    4: dict(name="cfg4 v1 bf16 65536 tok, d_model 4096, d_ff 16384, 64 experts",
            layer="v1", dtype="bf16", batch=32, length=2048, group=2048,
            M=4096, H=16384, E=64, cf=2.0),
    5: dict(name="cfg5 v2 bf16 32768 tok, d_model 2048, d_ff 8192, 8x16 experts",
            layer="v2", dtype="bf16", batch=32, length=1024, group=1024,
            M=2048, H=8192, E=[8, 16], cf=1.25, cf2=1.25),
}


def hparams_dict(cfg):
  return dict(
      moe_gating=cfg.get("gating", "top_2"), moe_switch_policy_train="argmax",
      moe_switch_policy_eval="argmax", moe_z_loss=None,
      moe_num_experts=cfg["E"], moe_loss_coef=1e-2,
      moe_hidden_size=cfg["H"], moe_group_size=cfg["group"],
      moe_min_expert_capacity=4, moe_capacity_factor_train=cfg["cf"],
      moe_capacity_factor_eval=cfg["cf"],
      moe_capacity_factor_second_level=cfg.get("cf2", 1.0),
      moe_use_second_place_loss=False, moe_second_policy_train="all",
      moe_second_policy_eval="all", moe_second_threshold_train=0.2,
      moe_second_threshold_eval=0.2,
      moe_dropout_rate=cfg.get("expert_dropout", 0.0),
      moe_use_experts_attention=False, moe_ntlb_top_k=4)


def normal_init(fan_in, seed):
  """N(0, 1/sqrt(fan_in)) generated on the device, one leading index at a time
  so that a 8 GiB variable never needs a float32 temporary of its full size."""
  import torch

  def init(sizes, dtype, device):
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    out = torch.empty(sizes, dtype=dtype, device=device)
    flat = out.reshape(sizes[0], -1) if len(sizes) > 2 else out.reshape(1, -1)
    for i in range(flat.shape[0]):
      row = torch.randn(flat.shape[1], generator=gen, device=device,
                        dtype=torch.float32)
      flat[i] = (row / math.sqrt(fan_in)).to(dtype)
    return out
  return init


def build(cfg, device, backward=False, operands="random"):
  """Builds the graph for `cfg` through the mtf-shaped API and lowers it once.
  With backward=True the graph also holds mtf.gradients of (outputs, loss)
  w.r.t. the tokens and the kernels.  Returns (lowering, x Tensor, y Tensor,
  loss Tensor)."""
  import torch
  import mesh_amd as mtf
  from mesh_amd.transformer import moe

  dt = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float32
  m, h = cfg["M"], cfg["H"]
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  gen = torch.Generator(device=device)
  gen.manual_seed(1)
  x_val = torch.randn((cfg["batch"], cfg["length"], m), generator=gen,
                      device=device, dtype=torch.float32).to(dt)
  dims = [mtf.Dimension("batch", cfg["batch"]),
          mtf.Dimension("length", cfg["length"]), mtf.Dimension("d_model", m)]
  hp = moe.HParams(**hparams_dict(cfg))
  vdt = mtf.VariableDType(dt, dt, dt)
  init = {}
  if cfg["layer"] == "v1":
    if cfg.get("skew"):
      # Zipf(s=1.2) rank profile scaled to 3.0, added to the router logits.  The
      # reference router has no bias term: feature 0 of every token is set to 1
      # and row 0 of the router kernel carries the bias.
      x_val[..., 0] = 1.0
    router = "moe/%s_gating/kernel" % cfg.get("gating", "top_2")
    init[router] = normal_init(m, 2)
    init["moe/wi/kernel"] = normal_init(m, 3)
    init["moe/wo/kernel"] = normal_init(h, 4)
  else:
    init["moe/outer_gating/kernel"] = normal_init(m, 2)
    init["moe/inner_gating/kernel"] = normal_init(m, 5)
    init["moe/wi/kernel"] = normal_init(m, 3)
    init["moe/wo/kernel"] = normal_init(h, 4)
  if operands != "random":
    # the same instruction stream and memory traffic on operands that do not
    # toggle the multipliers: what the chip's power limit costs this kernel
    zeros_init = lambda sizes, dtype, dev: torch.zeros(sizes, dtype=dtype,
                                                       device=dev)
    for name in list(init):
      if name.endswith("/wi/kernel") or name.endswith("/wo/kernel"):
        init[name] = zeros_init
    if operands == "zero_tokens":
      # zeros times zeros in the experts.  The router then sees equal logits
      # everywhere and sends every token to experts 0 and 1: only the padded
      # flop count (every slot row is multiplied, occupied or not) means
      # anything in this mode
      x_val = x_val * 0
  x = mtf.import_tf_tensor(mesh, x_val, mtf.Shape(dims))
  nonpadding = None
  if cfg.get("gating") == "expert_selection":
    # the reference's loss of this router sums `nonpadding`: every token counts
    nonpadding = mtf.import_tf_tensor(
        mesh, torch.ones(x_val.shape[:2], dtype=dt, device=device),
        mtf.Shape(dims[:2]))
  with mtf.variable_scope("moe"):
    if cfg["layer"] == "v1":
      y, loss = moe.transformer_moe_layer_v1(x, dims[-1], hp, True, vdt,
                                             nonpadding=nonpadding)
    else:
      y, loss = moe.transformer_moe_layer_v2(x, dims[-1], hp, True, vdt)
  if cfg.get("skew"):
    base = init[router]

    def skewed(sizes, dtype, dev):
      w = base(sizes, dtype, dev)
      perm = torch.randperm(sizes[1], generator=gen, device=dev) + 1
      w[0] = (3.0 * perm.double() ** -1.2).to(dtype)
      return w
    init[router] = skewed
  if backward:
    d_out = mtf.import_tf_tensor(
        mesh, torch.randn(x_val.shape, generator=gen, device=device,
                          dtype=torch.float32).to(dt), mtf.Shape(dims))
    mtf.gradients([y, loss],
                  [x] + [v.outputs[0] for v in graph.trainable_variables],
                  grad_ys=[d_out, None])
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl(device=device)},
                          initial_values=init)
  return lowering, x, y, loss


def build_block(cfg, device, backward=False):
  """The block of mesh_tensorflow/transformer/gin/models/lm_moe.gin:11-16
  (SelfAttention, MoE1D, SelfAttention, DenseReluDense; autoregressive, eval
  mode) around the layer of `cfg`: d_kv 128, d_model / 128 heads, d_ff and the
  experts' hidden size = cfg's H.  Variables keep their own initialisers
  (random normal).  With `backward`, also mtf.gradients of the output and the
  MoE loss w.r.t. the tokens and every variable.  Returns (lowering, x Tensor,
  y Tensor, None)."""
  import torch
  import mesh_amd as mtf
  from mesh_amd.transformer import moe, transformer, transformer_layers

  dt = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float32
  m = cfg["M"]
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  gen = torch.Generator(device=device)
  gen.manual_seed(1)
  x_val = torch.randn((cfg["batch"], cfg["length"], m), generator=gen,
                      device=device, dtype=torch.float32).to(dt)
  dims = [mtf.Dimension("batch", cfg["batch"]),
          mtf.Dimension("length", cfg["length"]), mtf.Dimension("d_model", m)]
  x = mtf.import_tf_tensor(mesh, x_val, mtf.Shape(dims))
  attention = (transformer_layers.SelfAttention,
               dict(num_heads=max(1, m // 128), key_value_size=128))
  stack = transformer.make_layer_stack(
      [attention,
       (moe.MoE1D, dict(num_experts=cfg["E"], hidden_size=cfg["H"],
                        group_size=cfg["group"], capacity_factor_eval=cfg["cf"],
                        second_policy_eval="all", second_policy_train="all")),
       attention,
       (transformer_layers.DenseReluDense, dict(hidden_size=cfg["H"]))],
      num_layers=1, block_scope=False)
  model = transformer.Unitransformer(stack, d_model=m, name="decoder",
                                     autoregressive=True)
  y, losses = model.call_layers(x, mtf.VariableDType(dt, dt, dt), mode="eval")
  if backward:
    d_out = mtf.import_tf_tensor(
        mesh, torch.randn(x_val.shape, generator=gen, device=device,
                          dtype=torch.float32).to(dt), mtf.Shape(dims))
    mtf.gradients([y] + list(losses),
                  [x] + [v.outputs[0] for v in graph.trainable_variables],
                  grad_ys=[d_out] + [None] * len(losses))
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl(device=device)})
  return lowering, x, y, None


def stage_model(cfg, kept_pairs, slots):
  """Algorithmic bytes / flops per step of each stage (v1 layer): what a
  perfect implementation has to move or compute."""
  b = 2 if cfg["dtype"] == "bf16" else 4
  t = cfg["batch"] * cfg["length"]
  m, h, e = cfg["M"], cfg["H"], cfg["E"]
  r = kept_pairs
  return {
      "router_logits": dict(bytes=t * m * b + m * e * b + t * e * 4),
      "top2_gating": dict(bytes=t * (4 * e + 26)),
      # fused projection + gating: the logits never reach HBM
      "router_top2_gating": dict(bytes=t * m * b + m * e * b + 26 * t),
      "switch_gating": dict(bytes=t * (4 * e + 26)),
      "router_switch_gating": dict(bytes=t * m * b + m * e * b + 26 * t),
      "ntlb_gating": dict(bytes=t * (4 * e + 26)),
      # experts choose tokens: slot records [G, E, C] and the token -> slot
      # table [G, S, E] int16
      "expert_choice_gating": dict(bytes=t * (4 * e + 2 * e) + 8 * slots),
      "slot_dispatch": dict(bytes=2 * slots * m * b + 4 * slots),
      "slot_combine": dict(bytes=slots * m * b + t * m * b + 2 * t * e
                           + 4 * slots),
      "dispatch": dict(bytes=t * m * b + r * m * b + 18 * t),
      "combine": dict(bytes=r * m * b + t * m * b + 26 * t),
      "expert_ffn": dict(flops=4 * r * m * h, padded_flops=4 * slots * m * h),
      # backward (only timed with --backward)
      "combine_backward": dict(bytes=t * m * b + 2 * r * m * b + 34 * t),
      "dispatch_backward": dict(bytes=r * m * b + t * m * b + t * e * 4 + 26 * t),
      "gating_backward": dict(bytes=t * (8 * e + 18)),
      "router_backward_weights": dict(bytes=t * m * b + t * e * 4),
      "expert_ffn_backward": dict(flops=8 * r * m * h,
                                  padded_flops=8 * slots * m * h),
  }


def cpu_baseline(cfg):
  """Times the CPU restatement of the reference lowering (dense one-hot
  dispatch/combine einsums, S x S cumsum matmul, per-expert matmuls) on a
  bounded sample: ONE group of the workload, with one expert's weight matrices
  shared by all experts so that host memory stays bounded."""
  import numpy as np
  from oracle import moe_oracle as O
  if cfg["layer"] != "v1":
    return None
  rng = np.random.default_rng(0)
  m, h, e, s = cfg["M"], cfg["H"], cfg["E"], cfg["group"]
  act = "bfloat16" if cfg["dtype"] == "bf16" else "float32"
  total_groups = cfg["batch"] * cfg["length"] // s
  # size the sample for roughly 10-30 s of host work (~7e11 flop/s measured on 16 cores)
  flops_per_group = 4.0 * e * max(4, min(s, int(s * cfg["cf"] / e))) * m * h
  n_groups = int(max(1, min(total_groups, round(1e13 / flops_per_group))))
  x = O.cast_act(rng.standard_normal((n_groups, s, m), dtype=np.float32), act)
  wg = (rng.standard_normal((m, e), dtype=np.float32) / np.sqrt(m))
  wi1 = O.cast_act(rng.standard_normal((1, m, h), dtype=np.float32)
                   / np.float32(np.sqrt(m)), act)
  wo1 = O.cast_act(rng.standard_normal((1, h, m), dtype=np.float32)
                   / np.float32(np.sqrt(h)), act)
  wi = np.broadcast_to(wi1, (e, m, h))
  wo = np.broadcast_to(wo1, (e, h, m))
  hp = O.HParams(**hparams_dict(cfg))
  threads = _blas_threads()
  t0 = time.perf_counter()
  O.moe_layer_v1(x, wg, wi, wo, hp, True, act, dense=True,
                 weights_are_cast=True)
  dt = time.perf_counter() - t0
  return dict(value=n_groups * s / dt, unit="tokens/s", cores=int(threads),
              kind="port",
              sample="%d of %d groups (%d tokens, all %d experts, dense "
                     "formulation, one expert's weights shared by all "
                     "experts), %.1f s"
                     % (n_groups, total_groups, n_groups * s, e, dt))


def cpu_baseline_full_cfg1():
  """The designated CPU configuration (config 1: fp32, 2048 tokens, d_model
  512, d_ff 2048, 8 experts) run WHOLE through the CPU restatement of the
  reference lowering: every group, every expert with weights of its own."""
  import numpy as np
  from oracle import moe_oracle as O
  cfg = CONFIGS[1]
  rng = np.random.default_rng(1)
  m, h, e, s = cfg["M"], cfg["H"], cfg["E"], cfg["group"]
  tokens = cfg["batch"] * cfg["length"]
  x = rng.standard_normal((tokens // s, s, m), dtype=np.float32)
  wg = rng.standard_normal((m, e), dtype=np.float32) / np.float32(np.sqrt(m))
  wi = rng.standard_normal((e, m, h), dtype=np.float32) / np.float32(np.sqrt(m))
  wo = rng.standard_normal((e, h, m), dtype=np.float32) / np.float32(np.sqrt(h))
  hp = O.HParams(**hparams_dict(cfg))
  best = None
  for _ in range(3):        # first pass pays the BLAS thread pool's start
    t0 = time.perf_counter()
    O.moe_layer_v1(x, wg, wi, wo, hp, True, "float32", dense=True,
                   weights_are_cast=True)
    dt = time.perf_counter() - t0
    best = dt if best is None else min(best, dt)
  return dict(value=tokens / best, unit="tokens/s", cores=_blas_threads(),
              kind="port", ms_per_step=best * 1e3,
              sample="the whole of %s (all %d tokens, %d groups, %d experts, "
                     "dense formulation), best of 3 passes"
                     % (cfg["name"], tokens, tokens // s, e))


def _blas_threads():
  threads = os.cpu_count()
  try:
    from threadpoolctl import threadpool_info
    blas = [p["num_threads"] for p in threadpool_info()
            if p.get("user_api") == "blas"]
    if blas:
      threads = max(blas)
  except Exception:  # pylint: disable=broad-except
    pass
  return int(threads)


class PowerSampler:
  """Samples the socket power, the shader clock and the violation counters of
  GPU 0 from a host thread (amdsmi) while a timed loop runs: the readings that
  say whether the chip sits at its power cap during the grouped GEMM."""

  def __init__(self, period_s=0.02):
    import threading
    import amdsmi
    self._amdsmi = amdsmi
    amdsmi.amdsmi_init()
    self._handle = amdsmi.amdsmi_get_processor_handles()[0]
    self._period = period_s
    self._stop = threading.Event()
    self._thread = threading.Thread(target=self._run, daemon=True)
    self.samples = []
    self.errors = []

  def _read(self):
    a, h = self._amdsmi, self._handle
    out = {}
    try:
      pw = a.amdsmi_get_power_info(h)
      for k in ("current_socket_power", "average_socket_power", "power_limit"):
        if k in pw and pw[k] != "N/A":
          out[k] = float(pw[k])
    except Exception as err:  # pylint: disable=broad-except
      self.errors.append("power_info: %r" % (err,))
    try:
      ck = a.amdsmi_get_clock_info(h, a.AmdSmiClkType.GFX)
      for k in ("clk", "cur_clk", "max_clk"):
        if k in ck and ck[k] != "N/A":
          out["gfx_" + k] = float(ck[k])
    except Exception as err:  # pylint: disable=broad-except
      self.errors.append("clock_info: %r" % (err,))
    return out

  def _run(self):
    while not self._stop.is_set():
      t = time.perf_counter()
      s = self._read()
      s["t"] = t
      self.samples.append(s)
      self._stop.wait(self._period)

  def static_info(self):
    """Power cap and violation (throttle) status, read once."""
    a, h = self._amdsmi, self._handle
    info = {}
    try:
      cap = a.amdsmi_get_power_cap_info(h)
      info["power_cap"] = {k: cap[k] for k in cap}
    except Exception as err:  # pylint: disable=broad-except
      info["power_cap_error"] = repr(err)
    try:
      v = a.amdsmi_get_violation_status(h)
      info["violation_status"] = {
          k: v[k] for k in v
          if isinstance(v[k], (int, float, str, bool)) and v[k] != "N/A"}
    except Exception as err:  # pylint: disable=broad-except
      info["violation_error"] = repr(err)
    return info

  def __enter__(self):
    self._thread.start()
    return self

  def __exit__(self, *exc):
    self._stop.set()
    self._thread.join()

  def summary(self, t0, t1):
    """Statistics of the samples taken inside [t0 + 20 %, t1] (the averaged
    power reading needs a moment to reach the loop's level)."""
    lo = t0 + 0.2 * (t1 - t0)
    inside = [s for s in self.samples if lo <= s["t"] <= t1]
    out = {"samples": len(inside), "window_s": t1 - lo}
    keys = sorted({k for s in inside for k in s if k != "t"})
    for k in keys:
      vals = sorted(s[k] for s in inside if k in s)
      if vals:
        out[k] = {"min": vals[0], "median": vals[len(vals) // 2],
                  "max": vals[-1], "mean": sum(vals) / len(vals)}
    if self.errors:
      out["errors"] = sorted(set(self.errors))[:4]
    return out


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=10)
  ap.add_argument("--warmup", type=int, default=3)
  ap.add_argument("--config", type=int, default=4, choices=sorted(CONFIGS))
  ap.add_argument("--gating", default="top_2",
                  choices=["top_2", "switch", "switch_max", "ntlb",
                           "expert_selection"],
                  help="router of the v1 configs (the benchmark definition "
                       "uses top_2)")
  ap.add_argument("--backward", action="store_true",
                  help="time forward + backward; the metric is "
                       "then named accordingly and is not the benchmark's")
  ap.add_argument("--block", action="store_true",
                  help="time the transformer block around the layer "
                       "(attention, MoE1D, attention, DenseReluDense; v1 "
                       "configs); not the benchmark's metric")
  ap.add_argument("--graph", action="store_true",
                  help="time replays of a recorded HIP graph of the step "
                       "(Lowering.capture) instead of eager runs; the per-stage "
                       "times still come from eager runs")
  ap.add_argument("--operands", default="random",
                  choices=["random", "zero_weights", "zero_tokens"],
                  help="diagnostic: zero expert weights (and tokens): the same "
                       "kernels and traffic without operand toggling, to read "
                       "the power limit off the clock; not the benchmark")
  ap.add_argument("--expert-dropout", type=float, default=0.0,
                  help="moe_dropout_rate of the layer (the dropout of the "
                       "experts' hidden tensor while training); not the "
                       "benchmark's configuration")
  ap.add_argument("--no-cpu-baseline", action="store_true")
  ap.add_argument("--router-alone", action="store_true",
                  help="diagnostic: after one step of the layer, time only its "
                       "router + gating launch, 3 x 200 launches back to back "
                       "(the chip has not been held at its power cap by the "
                       "expert GEMMs, as it has in the timed loop)")
  ap.add_argument("--power", action="store_true",
                  help="diagnostic: sample socket power and shader clock "
                       "(amdsmi, host thread) during the timed loop and add "
                       "them to the JSON line as `power`; use with enough "
                       "--steps for a few seconds of work")
  args = ap.parse_args()
  if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
    print("bench.py measures ONE GPU: this layer runs on a single-device mesh "
          "(no collectives are built); --gpus %d is not supported" % args.gpus,
          file=sys.stderr)
    sys.exit(2)

  import torch
  from mesh_amd import moe_hip
  cfg = dict(CONFIGS[args.config])
  if args.gating != "top_2":
    if cfg["layer"] != "v1":
      print("--gating applies to the v1 configs only", file=sys.stderr)
      sys.exit(2)
    cfg["gating"] = args.gating
    cfg["name"] += ", %s gating" % args.gating
  if args.expert_dropout:
    cfg["expert_dropout"] = args.expert_dropout
    cfg["name"] += ", moe_dropout_rate %g" % args.expert_dropout
  device = torch.device("cuda:0")
  torch.cuda.set_device(device)
  if args.router_alone and (cfg["layer"] != "v1" or args.block):
    print("--router-alone applies to the v1 layer configs", file=sys.stderr)
    sys.exit(2)
  if args.block and (cfg["layer"] != "v1" or args.gating != "top_2"):
    print("--block applies to the v1 configs, top_2", file=sys.stderr)
    sys.exit(2)
  if args.block:
    lowering, x, y, loss = build_block(cfg, device, args.backward)
  else:
    lowering, x, y, loss = build(cfg, device, args.backward,
                                 args.operands)            # first execution
  if args.router_alone:
    with moe_hip.StageTimer(keep_calls=True) as timer:
      lowering.run()
      torch.cuda.synchronize()
    names = [k for k in timer.calls if k.startswith("router_")]
    if len(names) != 1:
      print("--router-alone: the layer made no one-launch router call",
            file=sys.stderr)
      sys.exit(2)
    nbytes = stage_model(cfg, 0, 0)[names[0]]["bytes"]
    runs = [moe_hip.back_to_back_ms(timer.calls[names[0]], reps=200)
            for _ in range(3)]
    best = min(runs)
    print(json.dumps({
        "metric": "%s launch alone" % names[0], "unit": "ms",
        "value": best, "higher_is_better": False, "runs_ms": runs,
        "launches_per_run": 200, "algorithmic_bytes": nbytes,
        "GBps": nbytes / (best * 1e-3) / 1e9,
        "frac_hbm_peak": nbytes / (best * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "config": {"workload": cfg["name"]}}))
    return
  for _ in range(args.warmup):
    lowering.run()
  torch.cuda.synchronize()
  sampler = PowerSampler() if args.power else None
  power_before = sampler.static_info() if sampler else None
  with moe_hip.StageTimer(keep_calls=True) as timer:
    if sampler:
      sampler.__enter__()
    t0 = time.perf_counter()
    for _ in range(args.steps):
      lowering.run()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    if sampler:
      sampler.__exit__()
    stages = timer.totals()
    routings = timer.routing
  ms_per_step = (t1 - t0) * 1e3 / args.steps
  if args.graph:
    step = lowering.capture()
    for _ in range(args.warmup):
      step.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
      step.replay()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
  tokens = cfg["batch"] * cfg["length"]
  out_ok = bool(torch.isfinite(lowering.export_to_tf_tensor(y).float()).all())

  if args.block:
    # attention + MoE1D + attention + DenseReluDense: per-stage times only
    heads = max(1, cfg["M"] // 128)
    print(json.dumps({
        "metric": ("MoE transformer block fwd+bwd tokens/sec @1 GPU"
                   if args.backward
                   else "MoE transformer block fwd tokens/sec @1 GPU"),
        "value": tokens / (ms_per_step * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": cfg["dtype"],
        "data": "synthetic",
        "config": {"workload": "lm_moe block (attention, MoE1D, attention, "
                               "DenseReluDense) around " + cfg["name"],
                   "tokens": tokens, "heads": heads, "d_kv": 128,
                   "output_finite": out_ok},
        "roofline": None,
        "stages": {k: {"ms_per_step": v[1] / args.steps,
                       "launches_per_step": v[0] / args.steps}
                   for k, v in stages.items()},
        "cpu_baseline": None}))
    return
  result = {
      "metric": ("MoE layer fwd+bwd tokens/sec @1 GPU" if args.backward
                 else "MoE layer fwd tokens/sec @1 GPU"),
      "value": tokens / (ms_per_step * 1e-3), "unit": "tokens/s",
      "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
      "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
      "vs_baseline": None, "dtype": cfg["dtype"], "data": "synthetic",
      "config": {"workload": cfg["name"], "layer": cfg["layer"],
                 "tokens": tokens, "output_finite": out_ok,
                 "hip_graph": bool(args.graph), "operands": args.operands},
  }
  if cfg["layer"] == "v1":
    r = routings[-1]
    tile_rows = None
    if hasattr(r, "fill"):
      kept = int(r.fill.sum().item())
      slots = r.fill.numel() * r.capacity
      # compacted rows: an expert's occupied rows, rounded up to the 256-row
      # tiles the listed-tile kernels multiply whole
      used = r.fill.sum(dim=0)
      tile_rows = int(((used + 255) // 256 * 256).sum().item())
    else:
      # per-slot record: every slot holds a token, its weight may be 0
      slots = r.slot_token.numel()
      kept = slots
    model = stage_model(cfg, kept, slots)
    per_stage = {}
    for name, (calls, ms) in stages.items():
      ms_step = ms / args.steps
      entry = {"ms_per_step": ms_step, "launches_per_step": calls / args.steps}
      if "bytes" in model.get(name, {}):
        gbs = model[name]["bytes"] / (ms_step * 1e-3) / 1e9
        entry.update(algorithmic_bytes=model[name]["bytes"], GBps=gbs,
                     frac_hbm_peak=gbs / HBM_PEAK_GBS)
      per_stage[name] = entry
    # The router and combine launches once more, 50 of each back to back
    # between ONE pair of events: the launch's duration without the cost of an
    # event pair around every launch, which the per-step figures above carry
    # (several microseconds, a tenth of the router kernel).
    for name, call in timer.calls.items():
      entry = per_stage.get(name)
      if entry is None or entry["launches_per_step"] != 1.0:
        continue
      ms_b2b = moe_hip.back_to_back_ms(call)
      entry["back_to_back_ms"] = ms_b2b
      if "algorithmic_bytes" in entry:
        entry["frac_hbm_peak_back_to_back"] = (
            entry["algorithmic_bytes"] / (ms_b2b * 1e-3) / 1e9 / HBM_PEAK_GBS)
    # (with --expert-dropout and two choices per token the two expert GEMMs are
    # calls of their own, with the dropout between them)
    ffn_key = "expert_ffn" if "expert_ffn" in stages else "expert_linear"
    ffn_ms = stages[ffn_key][1] / args.steps
    # the expert FFN is two launches of the same grouped-GEMM kernel with the
    # same flop count; `achieved` prices the average launch
    flops_per_launch = model["expert_ffn"]["flops"] / 2
    achieved = flops_per_launch / (ffn_ms / 2 * 1e-3) / 1e12
    peak = MFMA_PEAK_TFLOPS[cfg["dtype"]]
    result["roofline"] = {
        "kernel": "grouped expert GEMM (expert_ffn, 2 launches/step)",
        "bound": "mfma", "achieved": achieved, "peak": peak,
        "unit": "TFLOP/s", "frac": achieved / peak,
        "traffic": (MEASURED_GEMM_TRAFFIC_BYTES.get(args.config)
                    if args.gating == "top_2" else None),
        "flops_per_launch": flops_per_launch,
        "avg_launch_ms": ffn_ms / 2,
        # fraction counting every row the kernels multiply: all slot rows,
        # or on compacted rows the tiles that hold occupied rows
        "padded_frac": ((model["expert_ffn"]["padded_flops"] / 2
                         * (tile_rows / slots if timer.compacted and tile_rows
                            else 1.0)
                         / (ffn_ms / 2 * 1e-3) / 1e12) / peak)}
    result["stages"] = per_stage
    if args.backward:
      bw_ms = stages["expert_ffn_backward"][1] / args.steps
      bw = model["expert_ffn_backward"]
      per_stage["expert_ffn_backward"].update(
          TFLOPs=bw["flops"] / (bw_ms * 1e-3) / 1e12,
          frac_mfma_peak=bw["flops"] / (bw_ms * 1e-3) / 1e12 / peak,
          padded_frac=(None if timer.compacted else
                       bw["padded_flops"] / (bw_ms * 1e-3) / 1e12 / peak))
    result["config"]["compacted_rows"] = bool(timer.compacted)
    result["config"].update(kept_pairs=kept, slots=slots,
                            capacity=r.capacity)
  else:
    # hierarchical layer: the expert FFN runs on the inner level's slots (the
    # last routing of a step), two launches of the grouped GEMM as in v1
    r = routings[-1]
    kept = int(r.fill.sum().item())
    slots = r.fill.numel() * r.capacity
    m, h = cfg["M"], cfg["H"]
    ffn_ms = stages["expert_ffn"][1] / args.steps
    peak = MFMA_PEAK_TFLOPS[cfg["dtype"]]
    flops_per_launch = 2.0 * kept * m * h
    achieved = flops_per_launch / (ffn_ms / 2 * 1e-3) / 1e12
    result["roofline"] = {
        "kernel": "grouped expert GEMM (expert_ffn, 2 launches/step)",
        "bound": "mfma", "achieved": achieved, "peak": peak,
        "unit": "TFLOP/s", "frac": achieved / peak, "traffic": None,
        "flops_per_launch": flops_per_launch, "avg_launch_ms": ffn_ms / 2,
        "padded_frac": (2.0 * slots * m * h / (ffn_ms / 2 * 1e-3) / 1e12) / peak}
    result["config"].update(kept_pairs=kept, slots=slots, capacity=r.capacity)
    result["stages"] = {k: {"ms_per_step": v[1] / args.steps,
                            "launches_per_step": v[0] / args.steps}
                        for k, v in stages.items()}
  # (the CPU restatement timed below is the top-2 layer's)
  if sampler:
    result["power"] = dict(sampler.summary(t0, t1), before=power_before,
                           after=sampler.static_info())
  no_cpu = args.no_cpu_baseline or args.backward or args.gating != "top_2"
  result["cpu_baseline"] = None if no_cpu else cpu_baseline(cfg)
  # the designated CPU configuration in full, beside the sample above
  result["cpu_baseline_full"] = None if no_cpu else cpu_baseline_full_cfg1()
  print(json.dumps(result))


if __name__ == "__main__":
  main()
