#!/usr/bin/env python3
"""Benchmark of the SNN-TC hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|cfg1|cfg2|cfg3|cfg4|cfg5|dense]

The last line of stdout is ONE short JSON record (under 1500 bytes); the per-kernel tables of every workload
go to stderr as a second JSON line (and to --detail-file).  A "step" is one pass of a workload over one synthetic batch that is already
resident in HBM.  The workloads are the five BASELINE configurations (and the north-star dense layer):

  cfg1   single SNN_dense 784->800 with bias, forward + backward, B=128.
  cfg2   3-layer SNN_dense MLP 784-800-800-10, B=256, full training step: forward,
         softmax-on-negative-time loss, snnfcgrad backward, SGD update.            (alias: mlp)
  cfg3   single SNN_conv 3x3 64->64 on 32x32, SAME, B=64, forward + backward.      (alias: conv)
  cfg4   CIFAR-shaped conv net training step, B=128.                               (alias: cifar)
  cfg5   ImageNet-shaped conv net, forward + loss + backward, B=32.                (alias: imagenet)
  dense  single SNN_dense 784->800 with bias, forward + backward, B=256.

The default, `--workload all`, times every one of them for K steps after W warm-up steps in this one
process.  The top-level fields of the record (value, ms_per_step, config, roofline, cpu_baseline) are
those of cfg5, the largest configuration that runs on one GPU; `per_config` holds one row per workload
(`per_config_fields` names the columns).  With a single workload named, the top level is that workload.

`value` is samples/s of the whole step.  `roofline` prices the kernel with the largest share of the
step against the MI355X peak that bounds it (algorithmic flops or bytes / its measured launch time,
HIP events recorded by the library on the launch stream); the detail line carries the same fraction for
every library kernel whose algorithmic work is defined.  `cpu_baseline` times the CPU restatement of
the reference's single-threaded host functors on this machine's cores, on a bounded sample.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "snntc-2023_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
VALU_PEAK_TFLOPS = 157.3     # MI355X fp32 vector peak (256 CU x 256 flop/clk x 2.4 GHz)

# rocprofv3 --pmc readings (HBM bytes per launch, share of clocks with a vector instruction issuing) cannot be
# taken from inside this script; they are carried from the tracked table that the profile summaries are written
# with, keyed by workload and kernel, and labelled with the commit they were measured at.
COUNTERS_FILE = os.path.join(ROOT, "profiles", "counters.json")


def _w_init(rng, fan_in, fan_out, bias=True):
    """N(4/fan_in, variance 1/fan_in); the bias row is drawn from the same law."""
    rows = fan_in + (1 if bias else 0)
    return (4.0 / fan_in + np.sqrt(1.0 / fan_in) * rng.standard_normal((rows, fan_out))).astype(np.float32)


# ------------------------------------------------------------------------------------------------
# workloads
# ------------------------------------------------------------------------------------------------
class Workload:
    name = ""
    key = ""
    batch = 0
    params = ()

    def step(self):
        raise NotImplementedError

    def layers(self):
        """[(layer module, its input tensor, whether the step asks for the input gradient, whether the
        tensor is already the padded one the conv op takes -- or "fed" when the layer before has written
        the padded tensor)], in forward order, for the accounting."""
        raise NotImplementedError

    extras = {}          # algorithmic bytes of the step's glue kernels (loss, SGD), by kernel name


class DenseLayerStep(Workload):
    """snnfc + snnfcgrad of one dense layer with bias (north-star dense layer; BASELINE config 1 at B=128)."""

    def __init__(self, torch, snn, dev, seed=0, batch=256, I=784, J=800, key="dense"):
        rng = np.random.default_rng(seed)
        self.torch, self.batch, self.snn, self.key = torch, batch, snn, key
        self.name = f"dense {I}->{J} bias B={batch} fwd+bwd"
        self.x = torch.from_numpy(np.exp(1.0 - rng.random((batch, I))).astype(np.float32)).to(dev)
        self.layer = snn.SNN_dense(I, J, weight=_w_init(rng, I, J)).to(dev)
        g = np.zeros((2 * batch, J), np.float32)
        g[:batch] = rng.standard_normal((batch, J))
        self.g = torch.from_numpy(g).to(dev)

    def step(self):
        l = self.layer
        y = self.snn.snnfc(self.x, l.weight.data, l.Params)
        return self.snn.snnfc_grad(self.g, self.x, l.weight.data, l.Params, y)

    def layers(self):
        return [(self.layer, self.x, True, False)]


class ConvLayerStep(Workload):
    """BASELINE config 3: snncv + snncvgrad, 3x3 64->64 at 32x32, SAME."""
    key = "cfg3"

    def __init__(self, torch, snn, dev, seed=0, batch=64, hw=32, C=64, Kc=64, k=3):
        rng = np.random.default_rng(seed)
        self.torch, self.batch, self.snn = torch, batch, snn
        self.name = f"conv {k}x{k} {C}->{Kc} @{hw}x{hw} SAME bias B={batch} fwd+bwd"
        x = torch.from_numpy(np.exp(rng.random((batch, hw, hw, C))).astype(np.float32)).to(dev)
        self.layer = snn.SNN_conv(C, Kc, k, 1, 'SAME', weight=_w_init(rng, k * k * C, Kc)).to(dev)
        self.xpad = self.layer.prepare_input(x).contiguous()
        g = np.zeros((2 * batch, hw, hw, Kc), np.float32)
        g[:batch] = rng.standard_normal((batch, hw, hw, Kc))
        self.g = torch.from_numpy(g).to(dev)

    def step(self):
        l = self.layer
        y = self.snn.snncv(self.xpad, l.weight.data, l.Params)
        return self.snn.snncv_grad(self.g, self.xpad, l.weight.data, l.Params, y)

    def layers(self):
        return [(self.layer, self.xpad, True, True)]          # the op is handed the padded tensor


class NetworkStep(Workload):
    """A layer stack of snntc_amd.networks: forward, softmax-on-negative-time loss, backward and, for the
    training configurations, one plain-SGD update of all layers."""

    def __init__(self, torch, snn, dev, key, title, spec, in_shape, classes, batch, train, seed=0, lr=1e-4):
        from snntc_amd import networks
        rng = np.random.default_rng(seed)
        self.torch, self.snn, self.key, self.batch, self.train, self.lr = torch, snn, key, batch, train, lr
        self.name = title
        x = rng.random((batch,) + tuple(in_shape)).astype(np.float32)
        self.z = torch.from_numpy(np.exp(1.0 - x)).to(dev)
        labels = rng.integers(0, classes, batch)
        self.onehot = torch.from_numpy(np.eye(classes, dtype=np.float32)[labels]).to(dev)
        self.net = networks.build(spec, rng=rng, chain=True).to(dev)     # no padding pass between chained layers
        self.params = self.net.weights()
        self._networks = networks
        n_w = float(sum(p.numel() for p in self.params))
        self.extras = {"softmax_time_loss": 12.0 * batch * classes}
        if train:
            self.extras["sgd_update"] = 12.0 * n_w

    def step(self):
        if self.train:
            return self._networks.sgd_train_step(self.net, self.z, self.onehot, self.lr)
        sample_loss, self.grads = self._networks.forward_backward(self.net, self.z, self.onehot)
        return sample_loss

    def layers(self):
        acts = []
        with self.torch.no_grad():
            self.net(self.z, keep=acts)
        out, mods = [], list(self.net)
        for i, (l, a) in enumerate(zip(mods, acts)):
            # a conv layer fed by the conv / pooling layer before it finds its input in its padded buffer
            fed = (i > 0 and isinstance(l, self.snn.SNN_conv) and l.padding == 'SAME'
                   and isinstance(mods[i - 1], (self.snn.SNN_conv, self.snn.SNN_maxpool2d)))
            out.append((l, a, i > 0, "fed" if fed else False))
        return out


def _make(key):
    def build(torch, snn, dev):
        from snntc_amd import networks as N
        if key == "cfg1":
            return DenseLayerStep(torch, snn, dev, batch=128, key="cfg1")
        if key == "dense":
            return DenseLayerStep(torch, snn, dev, batch=256, key="dense")
        if key == "cfg2":
            return NetworkStep(torch, snn, dev, "cfg2", "mlp 784-800-800-10 B=256 train step (fwd + loss + bwd + SGD)",
                               N.MLP, (784,), 10, 256, True)
        if key == "cfg3":
            return ConvLayerStep(torch, snn, dev)
        if key == "cfg4":
            return NetworkStep(torch, snn, dev, "cfg4", "cifar conv net B=128 train step (fwd + loss + bwd + SGD)",
                               N.CIFAR, (32, 32, 3), 10, 128, True)
        if key == "cfg5":
            return NetworkStep(torch, snn, dev, "cfg5", "imagenet-shaped conv net B=32 fwd+bwd",
                               N.IMAGENET, (224, 224, 3), 1000, 32, False)
        raise KeyError(key)
    return build


WORKLOADS = {k: _make(k) for k in ("cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "dense")}
ALIASES = {"mlp": "cfg2", "conv": "cfg3", "cifar": "cfg4", "imagenet": "cfg5", "dense128": "cfg1"}
ALL_ORDER = ("cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "dense")
HEADLINE = "cfg5"            # the largest BASELINE configuration that fits one GPU


# ------------------------------------------------------------------------------------------------
# HIP graph of one step
# ------------------------------------------------------------------------------------------------
def capture_step(torch, wl):
    """Captures wl.step() into a HIP graph (all launches of a step replayed with one call) and checks
    that replays reproduce eager steps bit for bit from the same starting weights.  Returns the graph,
    or None (with the reason) when capture or the check fails; the caller then times eager steps."""
    params = list(getattr(wl, "params", []))
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                wl.step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        start = [p.detach().clone() for p in params]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = wl.step()
        torch.cuda.synchronize()

        def restore():
            with torch.no_grad():
                for p, s0 in zip(params, start):
                    p.copy_(s0)

        def snapshot(res):
            vals = [p.detach().clone() for p in params]
            if isinstance(res, torch.Tensor):
                vals.append(res.detach().clone())
            elif isinstance(res, (tuple, list)):
                vals += [r.detach().clone() for r in res if isinstance(r, torch.Tensor)]
            return vals

        restore()
        eager = []
        for _ in range(3):
            eager.append(snapshot(wl.step()))
        restore()
        for i in range(3):
            graph.replay()
            torch.cuda.synchronize()
            got = snapshot(out)
            if len(got) != len(eager[i]) or not all(torch.equal(a, b) for a, b in zip(got, eager[i])):
                restore()
                return None, f"replay {i} differs from the eager step"
            _ = sum(float(v.sum()) for v in got[:1])      # eager work and a sync between replays
        restore()
        return graph, None
    except Exception as e:  # capture not possible on this stack: fall back to eager timing
        torch.cuda.synchronize()
        return None, f"{type(e).__name__}: {e}"


# ------------------------------------------------------------------------------------------------
# roofline accounting: algorithmic flops / bytes per kernel, summed over the layers of one step
# ------------------------------------------------------------------------------------------------
def account(torch, snn, layers, extras=None):
    """Per kernel name: algorithmic fp32 flops and HBM bytes of one step, from the causal-set sizes the
    forward actually produces.  Formulas (S segments of length I, J outputs, b = bias flag):
      steps = sum over (s,j) of consumed inputs + b ;   pairs = sum over fired (s,j) of (k + b)
      sort_segments : bytes 4*(in + 2*S*I), or 4*3*in when only the pixels' channels are sorted (merge path)
      merge_patches : bytes 4*(2*in + 2*S*I)                       flops 0 (comparisons are not flops)
      scan          : bytes 4*(2*S*I + (I+b)*J + 2*S*J)            flops 4*steps
      dX kernels    : bytes 4*(2*S*J + in + I*J + in)              flops 2*pairs
      grad_weight   : bytes 4*(2*S*J + in + (I+b)*J)               flops 3*pairs
      prep_upstream : bytes 4*(3*S*J + S*J + 2*I*J)                flops S*J   (carries the weight copy dX reads)
      fc_backward_narrow (J <= 16, the three above in one launch): bytes 4*(3*S*J + 2*in + 2*(I+b)*J), flops 5*pairs + S*J
      pad_time : bytes 4*(in + out) ;  min_pool / min_pool_grad : bytes 4*(in + 2*out)
    `in` is the op's input tensor (B*I dense, B*H*W*C padded image for conv)."""
    acc = {}

    def add(name, flops, nbytes):
        f, b = acc.get(name, (0.0, 0.0))
        acc[name] = (f + flops, b + nbytes)

    for layer, inp, want_dx, padded in layers:
        if isinstance(layer, snn.SNN_maxpool2d) or isinstance(layer, snn.SNN_globalminpool2d):
            with torch.no_grad():
                n_out = float(layer(inp).numel())
            add("min_pool", 0.0, 4.0 * (inp.numel() + 2.0 * n_out))
            add("min_pool_grad", 0.0, 4.0 * (inp.numel() + 2.0 * n_out))
            continue
        if not hasattr(layer, "weight"):
            continue
        W = layer.weight.data
        dense = isinstance(layer, snn.SNN_dense)
        with torch.no_grad():
            if dense:
                x_op = inp
                _, sz, _, ck = snn.snnfc(x_op, W, layer.Params, return_aux=True)
                max_t, bias = float(layer.Params[0]), int(layer.Params[5] > 1e-8)
                merged = False
            else:
                x_op = inp
                if padded is not True:               # a network layer: the layer pads (SAME) or crops (VALID) first;
                    x_op = layer.prepare_input(inp).contiguous()        # "fed": the layer before wrote the padded tensor
                    if x_op.numel() > inp.numel() and padded != "fed":
                        add("pad_time", 0.0, 4.0 * (inp.numel() + x_op.numel()))
                _, sz, _, ck = snn.snncv(x_op, W, layer.Params, return_aux=True)
                max_t, bias = float(layer.Params[0]), int(layer.Params[11] > 1e-8)
                merged = layer.C >= 32 and layer.C % 4 == 0 and layer.Kw >= 2
        S, I = sz.shape
        J = ck.shape[1]
        n_real = (sz <= np.float32(max_t) - np.float32(0.1)).sum(dim=1, keepdim=True)
        fired = ck >= 0
        consumed = torch.where(fired, ck, n_real.expand_as(ck).to(ck.dtype))
        steps = float((consumed + bias).sum().item())
        pairs = float((torch.where(fired, ck, torch.zeros_like(ck)) + bias * fired).sum().item())
        n_in = float(x_op.numel())
        if merged:
            add("sort_segments", 0.0, 4.0 * 3.0 * n_in)
            add("merge_patches", 0.0, 4.0 * (2.0 * n_in + 2.0 * S * I))
        else:
            add("sort_segments", 0.0, 4.0 * (n_in + 2.0 * S * I))
        add("scan", 4.0 * steps, 4.0 * (2.0 * S * I + (I + bias) * J + 2.0 * S * J))
        if dense and J <= 16:
            add("fc_backward_narrow", 5.0 * pairs + S * J, 4.0 * (3.0 * S * J + 2.0 * n_in + 2.0 * (I + bias) * J))
            continue
        if want_dx:
            add("fc_grad_input" if dense else "cv_grad_input", 2.0 * pairs, 4.0 * (2.0 * S * J + 2.0 * n_in + I * J))
        add("grad_weight", 3.0 * pairs, 4.0 * (2.0 * S * J + n_in + (I + bias) * J))
        add("prep_upstream", float(S * J), 4.0 * (4.0 * S * J + (2.0 * I * J if want_dx else 0.0)))
    for name, nbytes in (extras or {}).items():
        add(name, 0.0, nbytes)
    return acc


def roofline_for(name, flops, nbytes, avg_ms, launches_per_step):
    """Binding roofline of one kernel: the larger of bytes/HBM-peak and flops/VALU-peak."""
    t = avg_ms * 1e-3 * launches_per_step          # seconds per step spent in this kernel
    t_hbm = nbytes / (HBM_PEAK_GBS * 1e9)
    t_valu = flops / (VALU_PEAK_TFLOPS * 1e12)
    if t_valu >= t_hbm:
        ach = flops / t / 1e12
        return {"bound": "mfma", "achieved": ach, "peak": VALU_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": ach / VALU_PEAK_TFLOPS, "traffic": None,
                "note": "compute-bound: priced at the fp32 peak (157.3 TFLOP/s, equally the fp32 vector-ALU peak); "
                        "the path runs on the vector ALUs, no MFMA instruction is issued"}
    ach = nbytes / t / 1e9
    return {"bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": ach / HBM_PEAK_GBS,
            "traffic": None}


def carried_counters(workload_key, kernel):
    """Counter readings for (workload, kernel) from profiles/counters.json, or {}."""
    try:
        with open(COUNTERS_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return {}
    entry = dict(table.get("workloads", {}).get(workload_key, {}).get(kernel, {}))
    if "valu_busy" in entry:                 # share of the SIMDs' issue slots that hold a vector instruction
        entry["valu_busy"] = min(1.0, entry["valu_busy"])
    if entry:
        entry["source"] = f"profiles/counters.json at commit {table.get('commit', '?')}"
    return entry


# ------------------------------------------------------------------------------------------------
# CPU baseline: the reference's single-threaded host functors, restated (oracle *_host functions)
# ------------------------------------------------------------------------------------------------
_CPU_CONV_SPECS = {
    # conv layers (hw, C, Kc, kernel, stride), dense layers, sample batch
    "cfg3": ([(32, 64, 64, 3, 1)], (), 32),
    "cfg4": ([(32, 3, 32, 3, 1), (32, 32, 32, 3, 1), (16, 32, 64, 3, 1), (16, 64, 64, 3, 1), (8, 64, 128, 3, 1)],
             ((2048, 512), (512, 10)), 32),
    "cfg5": ([(224, 3, 64, 7, 2), (56, 64, 64, 3, 1), (56, 64, 64, 3, 1), (28, 64, 128, 3, 1), (28, 128, 128, 3, 1),
              (14, 128, 256, 3, 1), (14, 256, 256, 3, 1), (7, 256, 512, 3, 1), (7, 512, 512, 3, 1)],
             ((512, 1000),), 1),
}


def cpu_baseline(workload_key, seed=0):
    """Times the restated host functors (oracle *_host, gcc -O3, one thread) on a bounded sample of the
    workload: the same layer stack, forward + backward (+ SGD for the training steps), at batch B_cpu.
    Every host loop is linear in the batch, so samples/s does not depend on B_cpu."""
    from oracle import capi
    rng = np.random.default_rng(seed)
    if workload_key in ("cfg1", "cfg2", "dense"):
        sizes = (784, 800, 800, 10) if workload_key == "cfg2" else (784, 800)
        B = 128 if workload_key == "cfg1" else 256
        h = np.exp(1.0 - rng.random((B, sizes[0]))).astype(np.float32)
        ws = [_w_init(rng, sizes[i], sizes[i + 1]) for i in range(len(sizes) - 1)]
        p = capi.fc_params(1.0)
        reps = {"cfg1": 40, "cfg2": 10, "dense": 20}[workload_key]          # about 12 s of host work
        x0 = h
        t0 = time.perf_counter()
        for _ in range(reps):
            h = x0
            acts, outs = [], []
            for w in ws:
                acts.append(h)
                out = capi.fc_forward_host(h, w, p)
                outs.append(out)
                h = np.ascontiguousarray(out[:B])
            g = np.zeros_like(outs[-1]); g[:B] = rng.standard_normal((B, sizes[-1]))
            for w, a, out in zip(reversed(ws), reversed(acts), reversed(outs)):
                dx, dw, _ = capi.fc_backward_host(g, a, w, p, out)
                if workload_key == "cfg2":
                    w -= np.float32(1e-4) * dw
                g = np.zeros((2 * B, a.shape[1]), np.float32); g[:B] = dx
        n_samples = B * reps
        what = f"the same dense layer stack, {reps} steps"
    else:
        specs, dense, B = _CPU_CONV_SPECS[workload_key]
        t0 = time.perf_counter()
        for hw, C, Kc, k, st in specs:
            x = np.exp(rng.random((B, hw, hw, C))).astype(np.float32)
            pad = max((-(-hw // st) - 1) * st + k - hw, 0)         # SAME: the smaller half goes in front
            xpad = np.pad(x, ((0, 0), (pad // 2, pad - pad // 2), (pad // 2, pad - pad // 2), (0, 0)),
                          constant_values=np.float32(1e5))
            w = _w_init(rng, k * k * C, Kc)
            p = capi.cv_params(k, k, st, st, same=True, biasvolt=1.0)
            y = capi.cv_forward_host(xpad, w, p)
            out = np.concatenate((y, np.zeros_like(y)), axis=0)
            g = np.zeros_like(out); g[:B] = rng.standard_normal(y.shape)
            capi.cv_backward_host(g, xpad, w, p, out)
        for I, J in dense:
            xx = np.exp(1.0 - rng.random((B, I))).astype(np.float32)
            w = _w_init(rng, I, J)
            p = capi.fc_params(1.0)
            out = capi.fc_forward_host(xx, w, p)
            g = np.zeros_like(out); g[:B] = rng.standard_normal((B, J))
            capi.fc_backward_host(g, xx, w, p, out)
        n_samples = B
        what = "the same conv/dense layers (pooling and loss left out)"
    dt = time.perf_counter() - t0
    return {"value": n_samples / dt, "unit": "samples/s", "cores": 1, "kind": "port",
            "sample": f"B={B}, {what}, fwd+bwd; reference host functors restated in C, gcc -O3, 1 thread",
            "seconds": dt, "host_cpus": os.cpu_count()}


# ------------------------------------------------------------------------------------------------
def measure(torch, snn, _lib, dev, key, steps, warmup, use_graph=True, want_cpu=True):
    """Times one workload: W warm-up steps, exactly K timed steps (HIP-graph replays and eager launches of the
    same K steps; the faster launch path is the job's throughput), then a pass with the library's per-kernel
    HIP-event timing for the roofline figures."""
    wl = WORKLOADS[key](torch, snn, dev)
    graph, graph_note = capture_step(torch, wl) if use_graph else (None, "disabled by --no-graph")
    run_step = graph.replay if graph is not None else wl.step

    for _ in range(warmup):
        run_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run_step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / steps * 1e3

    # the same steps launched eagerly, after the same warm-up
    eager_ms_per_step = ms_per_step
    if graph is not None:
        for _ in range(warmup):
            wl.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            wl.step()
        torch.cuda.synchronize()
        eager_ms_per_step = (time.perf_counter() - t0) / steps * 1e3
    launch = "hip graph replay" if graph is not None else "eager"
    graph_ms_per_step = ms_per_step if graph is not None else None
    if graph is not None and eager_ms_per_step < ms_per_step:
        launch, ms_per_step = "eager", eager_ms_per_step

    # another pass over the same steps with the library's per-kernel HIP-event timing switched on
    prof_steps = min(steps, 50)
    _lib.profile_enable(True)
    for _ in range(prof_steps):
        wl.step()
    torch.cuda.synchronize()
    prof = _lib.profile_collect()
    _lib.profile_enable(False)
    snn.check_scan_health(dev)          # raises if a classifier-head scan gave up its bounded wait (NaN outputs)

    acc = account(torch, snn, wl.layers(), wl.extras)
    kernels = {}
    for name, (cnt, ms) in prof.items():
        kk = {"launches_per_step": cnt / prof_steps, "avg_us": ms / cnt * 1e3, "us_per_step": ms / prof_steps * 1e3}
        f, b = acc.get(name, (0.0, 0.0))
        kk["gflop_per_step"] = f / 1e9
        kk["mbyte_per_step"] = b / 1e6
        if f > 0.0 or b > 0.0:
            r = roofline_for(name, f, b, kk["avg_us"] * 1e-3, kk["launches_per_step"])
            kk["bound"], kk["frac"] = r["bound"], r["frac"]
        else:
            kk["bound"], kk["frac"] = None, None
        kernels[name] = kk
    dominant = max(kernels, key=lambda n: kernels[n]["us_per_step"])
    flops, nbytes = acc.get(dominant, (0.0, 0.0))
    k = kernels[dominant]
    roof = roofline_for(dominant, flops, nbytes, k["avg_us"] * 1e-3, k["launches_per_step"])
    carried = carried_counters(key, dominant)
    roof["traffic"] = carried.get("hbm_bytes_per_launch")
    roof["valu_busy"] = carried.get("valu_busy")
    roof["counters_source"] = carried.get("source")
    roof.update({"kernel": dominant, "avg_launch_us": k["avg_us"], "launches_per_step": k["launches_per_step"],
                 "algorithmic_flops_per_step": flops, "algorithmic_bytes_per_step": nbytes})

    res = {
        "value": wl.batch / (ms_per_step * 1e-3),
        "unit": "samples/s",
        "ms_per_step": ms_per_step,
        "config": {"workload": wl.name, "batch": wl.batch, "launch": launch, "graph_note": graph_note},
        "eager_ms_per_step": eager_ms_per_step,
        "graph_ms_per_step": graph_ms_per_step,
        "roofline": roof,
        "kernels": kernels,
        "library_kernel_us_per_step": sum(v["us_per_step"] for v in kernels.values()),
    }
    del graph, wl
    snn.ops.release_workspaces()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    if want_cpu:
        res["cpu_baseline"] = cpu_baseline(key)
        res["gpu_over_cpu"] = res["value"] / res["cpu_baseline"]["value"]
    return res


def _sig(v, digits=5):
    """Numbers rounded to `digits` significant digits (the record line is read by machines with a size limit)."""
    if isinstance(v, bool) or v is None or isinstance(v, (str, int)):
        return v
    if isinstance(v, float):
        return float(f"{v:.{digits}g}")
    if isinstance(v, dict):
        return {k: _sig(x, digits) for k, x in v.items()}
    if isinstance(v, (list, tuple)):
        return [_sig(x, digits) for x in v]
    return v


ROOFLINE_KEYS = ("bound", "kernel", "achieved", "peak", "unit", "frac", "traffic", "valu_busy", "avg_launch_us",
                 "launches_per_step", "algorithmic_flops_per_step", "algorithmic_bytes_per_step", "counters_source")
CPU_KEYS = ("value", "unit", "cores", "kind", "sample", "seconds", "host_cpus")
PER_CONFIG_FIELDS = ["ms_per_step", "samples_per_s", "dominant_kernel", "frac", "cpu_samples_per_s", "gpu_kernel_us"]
LINE_BUDGET = 1500           # bytes; the record line must stay below this


def headline(head, per_config, steps, warmup, device):
    """The one record line: the fields of the headline workload, its dominant kernel's roofline, its CPU
    baseline, and per workload a row of PER_CONFIG_FIELDS.  Everything else measure() returns (per-kernel
    tables) is printed elsewhere."""
    cfg = head["config"]
    result = {
        "metric": "SNN layer fwd+bwd samples/sec at 1 GPU; achieved HBM GB/s & % roofline",
        "value": head["value"],
        "unit": "samples/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": cfg["workload"], "batch": cfg["batch"], "launch": cfg["launch"], "device": device},
        "roofline": {k: head["roofline"].get(k) for k in ROOFLINE_KEYS},
    }
    if "cpu_baseline" in head:
        result["cpu_baseline"] = {k: head["cpu_baseline"].get(k) for k in CPU_KEYS}
    if per_config:
        result["per_config_fields"] = PER_CONFIG_FIELDS
        result["per_config"] = {
            key: [r["ms_per_step"], r["value"], r["roofline"]["kernel"], r["roofline"]["frac"],
                  r.get("cpu_baseline", {}).get("value"), r["library_kernel_us_per_step"]]
            for key, r in per_config.items()}
    return _sig(result)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", choices=["all"] + sorted(WORKLOADS) + sorted(ALIASES), default="all")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="time eager steps instead of HIP-graph replays")
    ap.add_argument("--calibration-copies", type=int, default=0,
                    help="first do this many plain 256 MiB device copies: a kernel of known traffic to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings of the same run by")
    ap.add_argument("--detail-file", default="", help="also write the per-kernel tables (JSON) to this file")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    import snntc_amd as snn
    from snntc_amd import _lib

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a ROCm GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    snn.init(dev)
    if args.calibration_copies > 0:
        src = torch.empty(256 * 1024 * 1024 // 4, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(args.calibration_copies):
            dst.copy_(src)                               # 256 MiB read + 256 MiB written per copy
        torch.cuda.synchronize()
        del src, dst

    keys = ALL_ORDER if args.workload == "all" else (ALIASES.get(args.workload, args.workload),)
    per_config = {}
    for key in keys:
        per_config[key] = measure(torch, snn, _lib, dev, key, args.steps, args.warmup,
                                  use_graph=not args.no_graph, want_cpu=not args.no_cpu_baseline)
    head = per_config[HEADLINE if args.workload == "all" else keys[0]]

    result = headline(head, per_config if args.workload == "all" else None, args.steps, args.warmup,
                      torch.cuda.get_device_name(0))
    # the per-kernel tables of every workload: one line on stderr (and a file, if asked for), so that the
    # last line of stdout stays a short record
    detail = json.dumps({"per_config": per_config})
    print(detail, file=sys.stderr)
    if args.detail_file:
        with open(args.detail_file, "w") as f:
            f.write(detail + "\n")
    sys.stderr.flush()
    print(json.dumps(result, separators=(",", ":")))


if __name__ == "__main__":
    main()
