#!/usr/bin/env python3
"""Benchmark of the SNN-TC hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload mlp|dense|conv|cifar|imagenet]

Prints ONE JSON line.  A "step" is one pass of the workload over one synthetic batch that is
already resident in HBM:

  mlp    (default; BASELINE config 2) 3-layer SNN_dense MLP 784-800-800-10, B=256, full training step:
         forward, softmax-on-negative-time loss, snnfcgrad backward, SGD update.
  dense  single SNN_dense 784->800 with bias, forward + backward, B=256 (north-star dense layer).
  conv   (BASELINE config 3) single SNN_conv 3x3 64->64 on 32x32, SAME, B=64, forward + backward.
  cifar  (BASELINE config 4) CIFAR-shaped conv net training step, B=128.

`value` is samples/s of the whole step.  `roofline` prices the kernel with the largest share of
the step against the MI355X peak that bounds it (algorithmic flops or bytes / its measured
launch time, HIP events recorded by the library on the launch stream).  `cpu_baseline` times the
CPU restatement of the reference's single-threaded host functors on this machine's cores.
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

# HBM bytes per launch of the scan kernel, measured with rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE (two runs,
# KiB per dispatch, FETCH_SIZE scaled by 2.0 and WRITE_SIZE by 1.0 as the plain 256 MiB device copies of
# --calibration-copies read on those counters); summary in profiles/scan_hbm_traffic_pmc.txt.  Counters cannot
# be read from inside this script, so the figures are carried here per workload (mlp: mean of its three launches).
MEASURED_SCAN_TRAFFIC_BYTES = {"mlp": 12.7e6, "conv": 341.3e6}
# Share of the scan kernel's clocks in which the vector ALUs issue (SQ_ACTIVE_INST_VALU * 4 / SIMDs / clocks,
# profiles/valu_utilisation_pmc.txt; mlp: mean of its three launches, 0.63 for the two 800-wide layers and 0.06 for
# the 10-wide head); the counter ratio saturates slightly above 1.
MEASURED_SCAN_VALU_BUSY = {"mlp": 0.44, "conv": 1.0}

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
VALU_PEAK_TFLOPS = 157.3     # MI355X fp32 vector peak (256 CU x 256 flop/clk x 2.4 GHz)


# ------------------------------------------------------------------------------------------------
# workloads
# ------------------------------------------------------------------------------------------------
def _w_init(rng, fan_in, fan_out, bias=True):
    """N(4/fan_in, variance 1/fan_in); the bias row is drawn from the same law."""
    rows = fan_in + (1 if bias else 0)
    return (4.0 / fan_in + np.sqrt(1.0 / fan_in) * rng.standard_normal((rows, fan_out))).astype(np.float32)


class Workload:
    name = ""
    batch = 0

    def step(self):
        raise NotImplementedError

    def layers(self):
        """[(kind, layer, input tensor fed to the op)] for the roofline accounting."""
        raise NotImplementedError


class MlpTrainStep(Workload):
    """BASELINE config 2."""
    name = "mlp 784-800-800-10 B=256 train step (fwd + loss + bwd + SGD)"

    def __init__(self, torch, snn, dev, seed=0, batch=256, sizes=(784, 800, 800, 10), lr=1e-4):
        rng = np.random.default_rng(seed)
        self.torch, self.batch, self.lr = torch, batch, lr
        x = rng.random((batch, 28, 28)).astype(np.float32)
        self.z = torch.from_numpy(np.exp(1.0 - x).reshape(batch, sizes[0])).to(dev)
        labels = rng.integers(0, sizes[-1], batch)
        self.onehot = torch.from_numpy(np.eye(sizes[-1], dtype=np.float32)[labels]).to(dev)
        self.net = [snn.SNN_dense(sizes[i], sizes[i + 1], weight=_w_init(rng, sizes[i], sizes[i + 1])).to(dev)
                    for i in range(len(sizes) - 1)]
        self.snn = snn
        self.params = [l.weight for l in self.net]

    def forward(self):
        h = self.z
        self.acts = []
        for l in self.net:
            self.acts.append(h)
            h = l(h)
        return h

    def step(self):
        torch = self.torch
        times = self.forward()
        # the loss kernel hands back the gradient of the batch mean: backpropagation starts from it
        sample_loss, dtimes = self.snn.softmax_time_loss(times.detach(), self.onehot)
        grads = torch.autograd.grad(times, self.params, grad_outputs=dtimes)
        self.snn.sgd_update(self.params, grads, self.lr)                      # SGD, all layers in one launch
        return sample_loss.mean()

    def layers(self):
        with self.torch.no_grad():
            self.forward()
        return [("dense", l, a) for l, a in zip(self.net, self.acts)]


class DenseLayerStep(Workload):
    """North-star dense layer: snnfc + snnfcgrad, 784->800, bias."""
    name = "dense 784->800 bias B=256 fwd+bwd"

    def __init__(self, torch, snn, dev, seed=0, batch=256, I=784, J=800):
        rng = np.random.default_rng(seed)
        self.torch, self.batch, self.snn = torch, batch, snn
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
        return [("dense", self.layer, self.x)]


class ConvLayerStep(Workload):
    """BASELINE config 3: snncv + snncvgrad, 3x3 64->64 at 32x32, SAME."""
    name = "conv 3x3 64->64 @32x32 SAME bias B=64 fwd+bwd"

    def __init__(self, torch, snn, dev, seed=0, batch=64, hw=32, C=64, Kc=64, k=3):
        rng = np.random.default_rng(seed)
        self.torch, self.batch, self.snn = torch, batch, snn
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
        return [("conv", self.layer, self.xpad)]


class CifarTrainStep(Workload):
    """BASELINE config 4."""
    name = "cifar conv net B=128 train step (fwd + loss + bwd + SGD)"

    def __init__(self, torch, snn, dev, seed=0, batch=128, lr=1e-4):
        rng = np.random.default_rng(seed)
        self.torch, self.batch, self.snn, self.lr = torch, batch, snn, lr
        x = rng.random((batch, 32, 32, 3)).astype(np.float32)
        self.z = torch.from_numpy(np.exp(1.0 - x)).to(dev)
        labels = rng.integers(0, 10, batch)
        self.onehot = torch.from_numpy(np.eye(10, dtype=np.float32)[labels]).to(dev)

        def conv(ci, co):
            return snn.SNN_conv(ci, co, 3, 1, 'SAME', weight=_w_init(rng, 9 * ci, co)).to(dev)

        def dense(i, o):
            return snn.SNN_dense(i, o, weight=_w_init(rng, i, o)).to(dev)

        pool = lambda: snn.SNN_maxpool2d(2, 2, 'SAME')
        self.net = [conv(3, 32), conv(32, 32), pool(), conv(32, 64), conv(64, 64), pool(), conv(64, 128), pool(),
                    "flatten", dense(2048, 512), dense(512, 10)]
        self.params = [l.weight for l in self.net if hasattr(l, "weight")]

    def forward(self, record=False):
        h = self.z
        self.acts = []
        for l in self.net:
            if isinstance(l, str):
                # "flatten", or the global min-time pool (earliest spike of every channel)
                h = h.amin(dim=(1, 2)) if l == "global_min" else h.reshape(h.shape[0], -1)
                continue
            if record and hasattr(l, "weight"):
                self.acts.append((l, h))
            h = l(h)
        return h

    def step(self):
        torch = self.torch
        times = self.forward()
        # the loss kernel hands back the gradient of the batch mean: backpropagation starts from it
        sample_loss, dtimes = self.snn.softmax_time_loss(times.detach(), self.onehot)
        grads = torch.autograd.grad(times, self.params, grad_outputs=dtimes)
        self.snn.sgd_update(self.params, grads, self.lr)                      # SGD, all layers in one launch
        return sample_loss.mean()

    def layers(self):
        with self.torch.no_grad():
            self.forward(record=True)
        out = []
        for l, a in self.acts:
            if isinstance(l, self.snn.SNN_conv):
                out.append(("conv", l, l.prepare_input(a).contiguous()))
            else:
                out.append(("dense", l, a))
        return out


class ImagenetFwdBwd(CifarTrainStep):
    """BASELINE config 5: forward + loss + backward (no weight update)."""
    name = "imagenet-shaped conv net B=32 fwd+bwd"

    def __init__(self, torch, snn, dev, seed=0, batch=32):
        rng = np.random.default_rng(seed)
        self.torch, self.batch, self.snn = torch, batch, snn
        x = rng.random((batch, 224, 224, 3)).astype(np.float32)
        self.z = torch.from_numpy(np.exp(1.0 - x)).to(dev)
        labels = rng.integers(0, 1000, batch)
        self.onehot = torch.from_numpy(np.eye(1000, dtype=np.float32)[labels]).to(dev)

        def conv(ci, co, k=3, s=1):
            return snn.SNN_conv(ci, co, k, s, 'SAME', weight=_w_init(rng, k * k * ci, co)).to(dev)

        pool = lambda: snn.SNN_maxpool2d(2, 2, 'SAME')
        self.net = [conv(3, 64, 7, 2), pool(),
                    conv(64, 64), conv(64, 64), pool(),
                    conv(64, 128), conv(128, 128), pool(),
                    conv(128, 256), conv(256, 256), pool(),
                    conv(256, 512), conv(512, 512),
                    "global_min", snn.SNN_dense(512, 1000, weight=_w_init(rng, 512, 1000)).to(dev)]
        self.params = [l.weight for l in self.net if hasattr(l, "weight")]

    def step(self):
        times = self.forward()
        sample_loss, dtimes = self.snn.softmax_time_loss(times.detach(), self.onehot)
        self.grads = self.torch.autograd.grad(times, self.params, grad_outputs=dtimes)
        return sample_loss.mean()


WORKLOADS = {"mlp": MlpTrainStep, "dense": DenseLayerStep, "conv": ConvLayerStep, "cifar": CifarTrainStep,
             "imagenet": ImagenetFwdBwd}


# ------------------------------------------------------------------------------------------------
# HIP graph of one step
# ------------------------------------------------------------------------------------------------
def capture_step(torch, wl):
    """Captures wl.step() into a HIP graph (all launches of a step replayed with one call) and checks
    that replays reproduce eager steps bit for bit from the same starting weights.  Returns the graph,
    or None (with the reason) when capture or the check fails; the caller then times eager steps."""
    params = getattr(wl, "params", [])
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
def account(torch, snn, layers):
    """Per kernel name: algorithmic fp32 flops and HBM bytes of one step, from the causal-set sizes the
    forward actually produces.  Formulas (S segments of length I, J outputs, b = bias flag):
      steps = sum over (s,j) of consumed inputs + b ;   pairs = sum over fired (s,j) of (k + b)
      sort_segments : bytes 4*(in + 2*S*I)                         flops 0 (comparisons are not flops)
      scan          : bytes 4*(2*S*I + (I+b)*J + 2*S*J)            flops 4*steps
      dX kernels    : bytes 4*(2*S*J + in + I*J + in)              flops 2*pairs
      grad_weight   : bytes 4*(2*S*J + in + (I+b)*J)               flops 3*pairs
      prep_upstream : bytes 4*(3*S*J + 2*S*J + 2*I*J)              flops S*J   (carries the weight copy dX reads)
    `in` is the op's input tensor (B*I dense, B*H*W*C padded image for conv)."""
    acc = {}

    def add(name, flops, nbytes):
        f, b = acc.get(name, (0.0, 0.0))
        acc[name] = (f + flops, b + nbytes)

    for kind, layer, inp in layers:
        W = layer.weight.data
        with torch.no_grad():
            if kind == "dense":
                _, sz, _, ck = snn.snnfc(inp, W, layer.Params, return_aux=True)
                max_t, bias = float(layer.Params[0]), int(layer.Params[5] > 1e-8)
            else:
                _, sz, _, ck = snn.snncv(inp, W, layer.Params, return_aux=True)
                max_t, bias = float(layer.Params[0]), int(layer.Params[11] > 1e-8)
        S, I = sz.shape
        J = ck.shape[1]
        n_real = (sz <= np.float32(max_t) - np.float32(0.1)).sum(dim=1, keepdim=True)
        fired = ck >= 0
        consumed = torch.where(fired, ck, n_real.expand_as(ck).to(ck.dtype))
        steps = float((consumed + bias).sum().item())
        pairs = float((torch.where(fired, ck, torch.zeros_like(ck)) + bias * fired).sum().item())
        n_in = float(inp.numel())
        add("sort_segments", 0.0, 4.0 * (n_in + 2.0 * S * I))
        add("scan", 4.0 * steps, 4.0 * (2.0 * S * I + (I + bias) * J + 2.0 * S * J))
        add("fc_grad_input" if kind == "dense" else "cv_grad_input", 2.0 * pairs,
            4.0 * (2.0 * S * J + 2.0 * n_in + I * J))
        add("grad_weight", 3.0 * pairs, 4.0 * (2.0 * S * J + n_in + (I + bias) * J))
        add("prep_upstream", float(S * J), 4.0 * (5.0 * S * J + 2.0 * I * J))     # with the weight copy for dX
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


# ------------------------------------------------------------------------------------------------
# CPU baseline: the reference's single-threaded host functors, restated (oracle *_host functions)
# ------------------------------------------------------------------------------------------------
def cpu_baseline(workload_key, seed=0):
    """Times the restated host functors (oracle *_host, gcc -O3, one thread) on a bounded sample of the
    workload: the same layer stack, forward + backward (+ SGD for the training steps), at batch B_cpu.
    Every host loop is linear in the batch, so samples/s does not depend on B_cpu."""
    from oracle import capi
    rng = np.random.default_rng(seed)
    t0 = time.perf_counter()
    if workload_key in ("mlp", "dense"):
        sizes = (784, 800, 800, 10) if workload_key == "mlp" else (784, 800)
        B = 256
        h = np.exp(1.0 - rng.random((B, sizes[0]))).astype(np.float32)
        ws = [_w_init(rng, sizes[i], sizes[i + 1]) for i in range(len(sizes) - 1)]
        p = capi.fc_params(1.0)
        reps = 10 if workload_key == "mlp" else 20          # about 12 s of host work
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
                w -= np.float32(1e-4) * dw
                g = np.zeros((2 * B, a.shape[1]), np.float32); g[:B] = dx
        what = f"the same dense layer stack, {reps} steps"
    else:
        # conv layers (hw, C, Kc, kernel, stride); pooling and loss are left out of the CPU sample
        if workload_key == "conv":
            specs, dense, B = [(32, 64, 64, 3, 1)], (), 32
        elif workload_key == "cifar":
            specs = [(32, 3, 32, 3, 1), (32, 32, 32, 3, 1), (16, 32, 64, 3, 1), (16, 64, 64, 3, 1), (8, 64, 128, 3, 1)]
            dense, B = ((2048, 512), (512, 10)), 32
        else:  # imagenet
            specs = [(224, 3, 64, 7, 2), (56, 64, 64, 3, 1), (56, 64, 64, 3, 1), (28, 64, 128, 3, 1),
                     (28, 128, 128, 3, 1), (14, 128, 256, 3, 1), (14, 256, 256, 3, 1), (7, 256, 512, 3, 1),
                     (7, 512, 512, 3, 1)]
            dense, B = ((512, 1000),), 1
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
        what = "the same conv/dense layers (pooling and loss left out)"
    dt = time.perf_counter() - t0
    n_samples = B * (reps if workload_key in ("mlp", "dense") else 1)
    return {"value": n_samples / dt, "unit": "samples/s", "cores": 1, "kind": "port",
            "sample": f"B={B} through {what}, fwd+bwd, reference host functors restated in C (gcc -O3), 1 thread",
            "seconds": dt, "host_cpus": os.cpu_count()}


# ------------------------------------------------------------------------------------------------
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="mlp")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="time eager steps instead of HIP-graph replays")
    ap.add_argument("--calibration-copies", type=int, default=0,
                    help="first do this many plain 256 MiB device copies: a kernel of known traffic to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings of the same run by")
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
    if args.calibration_copies > 0:
        src = torch.empty(256 * 1024 * 1024 // 4, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(args.calibration_copies):
            dst.copy_(src)                               # 256 MiB read + 256 MiB written per copy
        torch.cuda.synchronize()
        del src, dst
    wl = WORKLOADS[args.workload](torch, snn, dev)

    graph, graph_note = (None, "disabled by --no-graph") if args.no_graph else capture_step(torch, wl)
    run_step = graph.replay if graph is not None else wl.step

    for _ in range(args.warmup):
        run_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3

    # the same steps launched eagerly, for reference
    for _ in range(3):
        wl.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        wl.step()
    torch.cuda.synchronize()
    eager_ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    # The same K steps were timed both ways; the job's throughput is that of the faster launch path
    # (graph replay saves host time per launch, a fast host can keep the queue full without it).
    launch = "hip graph replay" if graph is not None else "eager"
    graph_ms_per_step = ms_per_step if graph is not None else None
    if graph is not None and eager_ms_per_step < ms_per_step:
        launch, ms_per_step, dt = "eager", eager_ms_per_step, eager_ms_per_step * 1e-3 * args.steps

    # second pass over the same steps with the library's per-kernel HIP-event timing switched on
    _lib.profile_enable(True)
    for _ in range(args.steps):
        wl.step()
    torch.cuda.synchronize()
    prof = _lib.profile_collect()
    _lib.profile_enable(False)

    kernels = {}
    for name, (cnt, ms) in prof.items():
        kernels[name] = {"launches_per_step": cnt / args.steps, "avg_us": ms / cnt * 1e3,
                         "us_per_step": ms / args.steps * 1e3}
    acc = account(torch, snn, wl.layers())
    dominant = max(kernels, key=lambda n: kernels[n]["us_per_step"])
    flops, nbytes = acc.get(dominant, (0.0, 0.0))
    k = kernels[dominant]
    roof = roofline_for(dominant, flops, nbytes, k["avg_us"] * 1e-3, k["launches_per_step"])
    if dominant == "scan":
        roof["traffic"] = MEASURED_SCAN_TRAFFIC_BYTES.get(args.workload)
        roof["valu_busy"] = MEASURED_SCAN_VALU_BUSY.get(args.workload)
    roof.update({"kernel": dominant, "avg_launch_us": k["avg_us"], "launches_per_step": k["launches_per_step"],
                 "algorithmic_flops_per_step": flops, "algorithmic_bytes_per_step": nbytes})
    for name, kk in kernels.items():
        f, b = acc.get(name, (0.0, 0.0))
        kk["gflop_per_step"] = f / 1e9
        kk["mbyte_per_step"] = b / 1e6

    result = {
        "metric": "SNN layer fwd+bwd samples/sec at 1 GPU; achieved HBM GB/s & % roofline",
        "value": wl.batch / (dt / args.steps),
        "unit": "samples/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": wl.name, "batch": wl.batch, "device": torch.cuda.get_device_name(0),
                   "launch": launch, "graph_note": graph_note},
        "eager_ms_per_step": eager_ms_per_step,
        "graph_ms_per_step": graph_ms_per_step,
        "roofline": roof,
        "kernels": kernels,
        "library_kernel_us_per_step": sum(v["us_per_step"] for v in kernels.values()),
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.workload)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
