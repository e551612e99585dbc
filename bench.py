#!/usr/bin/env python3
"""Benchmark of the fused 4-bit AdamW step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama3-8b]

One "step" is one `optimizer.step()` over the whole synthetic parameter set: one
multi-tensor launch of the fused 4-bit kernel per batch of 48 tensors plus one launch of
the non-quantized kernel for the tensors of at most 4096 elements.  Inputs are resident in
HBM before the timed region starts.  Prints ONE JSON line:

  value         parameters updated per second over the timed region (wall clock
                around K steps, synchronised on both sides)
  roofline      the fused kernel against HBM: algorithmic bytes per launch divided
                by its average duration, measured with events on the launch stream
                inside the same timed region; `traffic` = HBM bytes per launch from
                hardware counters (profiles/hbm_traffic.json), null when the kernel
                sources have changed since they were read
  cpu_baseline  the CPU oracle (vectorised torch restatement of the reference's
                PyTorch path) timed on this machine's host cores on a bounded
                sample of the same workload
  configs       (default run only) the other benchmark configurations and the step's
                variants, each timed the same way in this same process: step time,
                kernel time, launches, fraction of peak, host time per step, and for
                the block-scaled ones the fraction of the `ceiling` probe with their
                element types (measured on 2^30 elements, whatever the configuration's size)
  ceiling       what this GPU's memory system gives kernels that move the step's bytes
                in the step's access pattern without its arithmetic (libq4probe.so): a
                plain copy, a read-only stream and the step's seven streams; the
                roofline entries carry `frac_of_ceiling` against the last of these
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

HP = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)


def llama3_8b_shapes():
    shapes = [("embed_tokens", (128256, 4096)), ("lm_head", (128256, 4096))]
    for i in range(32):
        shapes += [
            (f"layers.{i}.q_proj", (4096, 4096)),
            (f"layers.{i}.k_proj", (1024, 4096)),
            (f"layers.{i}.v_proj", (1024, 4096)),
            (f"layers.{i}.o_proj", (4096, 4096)),
            (f"layers.{i}.gate_proj", (14336, 4096)),
            (f"layers.{i}.up_proj", (14336, 4096)),
            (f"layers.{i}.down_proj", (4096, 14336)),
            (f"layers.{i}.input_layernorm", (4096,)),
            (f"layers.{i}.post_attention_layernorm", (4096,)),
        ]
    shapes.append(("norm", (4096,)))
    return shapes


def llama2_13b_shapes():
    shapes = [("embed_tokens", (32000, 5120)), ("lm_head", (32000, 5120))]
    for i in range(40):
        shapes += [(f"layers.{i}.{n}_proj", (5120, 5120)) for n in "qkvo"]
        shapes += [
            (f"layers.{i}.gate_proj", (13824, 5120)),
            (f"layers.{i}.up_proj", (13824, 5120)),
            (f"layers.{i}.down_proj", (5120, 13824)),
            (f"layers.{i}.input_layernorm", (5120,)),
            (f"layers.{i}.post_attention_layernorm", (5120,)),
        ]
    return shapes


def gpt2_small_shapes():
    shapes = [("wte", (50257, 768)), ("wpe", (1024, 768))]
    for i in range(12):
        shapes += [
            (f"h.{i}.ln_1.weight", (768,)), (f"h.{i}.ln_1.bias", (768,)),
            (f"h.{i}.attn.c_attn.weight", (768, 2304)), (f"h.{i}.attn.c_attn.bias", (2304,)),
            (f"h.{i}.attn.c_proj.weight", (768, 768)), (f"h.{i}.attn.c_proj.bias", (768,)),
            (f"h.{i}.ln_2.weight", (768,)), (f"h.{i}.ln_2.bias", (768,)),
            (f"h.{i}.mlp.c_fc.weight", (768, 3072)), (f"h.{i}.mlp.c_fc.bias", (3072,)),
            (f"h.{i}.mlp.c_proj.weight", (3072, 768)), (f"h.{i}.mlp.c_proj.bias", (768,)),
        ]
    shapes += [("ln_f.weight", (768,)), ("ln_f.bias", (768,))]
    return shapes


WORKLOADS = {
    # name: (shapes, param dtype, grad dtype, grad distribution, description)
    "llama3-8b": (llama3_8b_shapes, "float32", "bfloat16", "student_t",
                  "BASELINE.json configs[3]: Llama-3-8B parameter set, 291 tensors, fp32 master "
                  "params, bf16 grads, 4-bit m/v, block 128"),
    "llama2-13b": (llama2_13b_shapes, "bfloat16", "bfloat16", "student_t",
                   "BASELINE.json configs[4]: Llama-2-13B-shaped parameter set, 362 tensors, bf16 "
                   "params, bf16 grads, 4-bit m/v, block 128"),
    "gpt2-small": (gpt2_small_shapes, "float32", "float32", "normal_outliers",
                   "BASELINE.json configs[1]: GPT-2-small parameter set, 148 tensors, fp32 params and "
                   "grads, 4-bit m/v, block 128"),
    "single-4096": (lambda: [("w", (4096, 4096))], "float32", "float32", "normal_outliers",
                    "BASELINE.json configs[0]: single fp32 4096x4096 tensor"),
    # one 2^30-element tensor: the kernel alone, free of the parameter sets' launch mix
    # (--param-dtype / --grad-dtype choose the kernel variant)
    "single-2p30": (lambda: [("w", (1 << 30,))], "float32", "bfloat16", "student_t",
                    "one tensor of 2^30 elements (kernel-only workload, not a BASELINE.json configuration)"),
}
DTYPE_NAMES = ("float32", "bfloat16", "float16")


def make_grad(torch, shape, dist, gen, device, dtype):
    n = 1
    for s in shape:
        n *= s
    if dist == "student_t":
        z = torch.randn(n, generator=gen, device=device)
        c = torch.zeros(n, device=device)
        for _ in range(3):
            c += torch.randn(n, generator=gen, device=device).square_()
        g = z * torch.rsqrt(c / 3.0) * 1e-4
    else:
        g = torch.randn(n, generator=gen, device=device) * 1e-3
        mask = torch.rand(n, generator=gen, device=device) < 1e-3
        sign = torch.where(torch.rand(n, generator=gen, device=device) < 0.5, -1.0, 1.0)
        g = torch.where(mask, sign * 1e-1, g)
    return g.to(dtype).view(shape)


def bytes_per_param(p_dtype, g_dtype):
    """Algorithmic HBM bytes per parameter of the fused kernel: p read + write, g read,
    one nibble of each moment read + write, two fp32 scales per 128 read + write."""
    pb = 4 if p_dtype == "float32" else 2
    gb = 4 if g_dtype == "float32" else 2
    return 2 * pb + gb + 2 * (0.5 + 0.5) + 2 * 2 * 4 / 128.0


def cpu_baseline(torch, params, grads_set, hp, budget_s=20.0):
    """Times the torch-CPU oracle on the first quantized tensors of the workload until
    about budget_s seconds of CPU work have been spent."""
    from oracle import q4_oracle_torch as ot
    done_params, spent, used = 0, 0.0, {}
    for p, g in zip(params, grads_set):
        if p.numel() <= 4096 or p.numel() > (1 << 26):
            continue
        pc = p.detach().float().cpu().reshape(-1)
        gc = g.detach().cpu().reshape(-1)
        n = pc.numel()
        mc = torch.zeros((n + 1) // 2, dtype=torch.uint8)
        vc = mc.clone()
        ms = torch.zeros((n + 127) // 128)
        vs = ms.clone()
        ot.step_quant(pc[:4096], gc[:4096], mc[:2048], vc[:2048], ms[:32], vs[:32], step=1,
                      beta1=hp["betas"][0], beta2=hp["betas"][1], lr=hp["lr"],
                      weight_decay=hp["weight_decay"], eps=hp["eps"])  # warm caches
        for step in (1, 2):
            t0 = time.perf_counter()
            pc, mc, vc, ms, vs = ot.step_quant(pc, gc, mc, vc, ms, vs, step=step,
                                               beta1=hp["betas"][0], beta2=hp["betas"][1],
                                               lr=hp["lr"], weight_decay=hp["weight_decay"],
                                               eps=hp["eps"])
            spent += time.perf_counter() - t0
            done_params += n
        key = "x".join(str(d) for d in p.shape)
        used[key] = used.get(key, 0) + 1
        if spent >= budget_s:
            break
    return {
        "value": done_params / spent if spent else None,
        "unit": "params/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": "torch-CPU 3-pass oracle, 2 steps each on the workload's first tensors: "
                  + ", ".join(f"{n} of {k}" for k, n in used.items())
                  + f" ({done_params / 2 / 1e6:.0f}M params, {spent:.1f} s)",
    }


def build_inputs(torch, device, shapes, p_dtype, g_dtype, dist, grad_sets):
    """Parameters and pre-generated gradient sets of one workload, resident on the device."""
    gen = torch.Generator(device=device).manual_seed(0)
    params = []
    for _, shape in shapes:
        p = (torch.randn(shape, generator=gen, device=device) * 0.02).to(p_dtype)
        p = torch.nn.Parameter(p, requires_grad=True)
        if g_dtype != p_dtype:
            p.grad_dtype = g_dtype  # e.g. an fp32 master parameter with a bf16 gradient
        params.append(p)
    grads = [[make_grad(torch, shape, dist, gen, device, g_dtype) for _, shape in shapes]
             for _ in range(max(1, grad_sets))]
    return params, grads


def run_config(torch, params, grad_sets, p_dtype_s, g_dtype_s, steps, warmup, variance_scale="group",
               round_type="real-nearest", clip="none", host_burst=True, param_update="auto"):
    """W warm-up steps, then exactly K timed steps between two synchronisations, with a fresh
    optimizer over `params`.  Returns the measurements of the timed region.  host_burst=False
    leaves out the extra steps that measure the host time of step() (host_ms_per_step is then
    None): W + K steps run and no others, which a counter profile of the run relies on."""
    from quantfour_adamw_cuda_amd import AdamWFused_QuantFour
    opt = AdamWFused_QuantFour(params, variance_scale_type=variance_scale, round_type=round_type, seed=0,
                               param_update=param_update, **HP)
    opt.kernel_timing = []  # (kind, start event, end event) per launch
    host_s = [0.0]

    def one_step(i):
        gs = grad_sets[i % len(grad_sets)]
        for p, g in zip(params, gs):
            p.grad = g
        h0 = time.perf_counter()
        if clip == "fused":
            opt.step(grad_scale=1.0 / 1024.0, max_grad_norm=1.0)
        elif clip == "separate":
            torch._foreach_mul_(gs, 1.0 / 1024.0)
            torch.nn.utils.clip_grad_norm_(params, 1.0, foreach=True)
            opt.step()
        else:
            opt.step()
        host_s[0] += time.perf_counter() - h0

    for i in range(warmup):
        one_step(i)
    torch.cuda.synchronize()
    opt.kernel_timing.clear()
    host_s[0] = 0.0

    t0 = time.perf_counter()
    for i in range(steps):
        one_step(warmup + i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    kernel_timing, opt.kernel_timing = opt.kernel_timing, None

    # one entry per step: the step's fused launches (one kernel per batch of up to 48
    # tensors, back to back on the stream) between two events
    fused_ms = [s.elapsed_time(e) for kind, s, e in kernel_timing if kind.startswith("fused_4bit")]
    avg_kernel_s = sum(fused_ms) / steps / 1e3
    rank1 = [p for p in params if opt.state[p]["variance_qstate"]["overhead"].get("max_dims") is not None]
    grouped = sum(1 for p in params if p.numel() > 4096) - len(rank1)
    # kernels per step: one per batch of 48 block-scaled tensors; statistics + update +
    # commit per batch of 32 rank-1 tensors
    launches_per_step = -(-grouped // 48) + 3 * -(-len(rank1) // 32)

    # Host time of step(): a burst of a few more steps issued into the drained queue, without
    # the timing events (the first two of them untimed: the first launch after an idle
    # period costs more).  Inside the timed region the device is the slower side, the launch
    # queue fills, and the time a launch call spends waiting for room would be counted as the
    # host's; the burst stays under 200 launches for the same reason.
    host_ms_per_step = None
    if host_burst:
        small = sum(1 for p in params if p.numel() <= 4096)
        burst = max(2, min(steps, 16, 192 // (launches_per_step + -(-small // 80)) - 2))
        for i in range(2 + burst):
            if i == 2:
                host_s[0] = 0.0
            one_step(warmup + steps + i)
        host_ms_per_step = host_s[0] / burst * 1e3
        torch.cuda.synchronize()

    quant_params = sum(p.numel() for p in params if p.numel() > 4096)
    algo_bytes = quant_params * bytes_per_param(p_dtype_s, g_dtype_s)
    if rank1:
        # the statistics pass reads g and the second moment's codes once more; no block scales
        # for the second moment, row and column maxima instead (read twice, written twice)
        gb = 4 if g_dtype_s == "float32" else 2
        n1 = sum(p.numel() for p in rank1)
        algo_bytes += n1 * (gb + 0.5 - 2 * 4 / 128.0) + sum(16 * (p.shape[0] + p.shape[1]) for p in rank1)
    m = dict(elapsed=elapsed, steps=steps, ms_per_step=elapsed / steps * 1e3, kernel_s=avg_kernel_s,
             launches_per_step=launches_per_step, algo_bytes=algo_bytes, rank1=len(rank1),
             quant_params=quant_params, total_params=sum(p.numel() for p in params),
             host_ms_per_step=host_ms_per_step)
    norm_ms = [s.elapsed_time(e) for kind, s, e in kernel_timing if kind == "grad_norm"]
    if norm_ms:
        m["norm_s"] = sum(norm_ms) / steps / 1e3
    return m


def update_form_of(param_update, p_dtype_s, variance_scale, round_type):
    """which form of the parameter update a run's quantized kernels compute (the library's
    "auto" rule: exact for fp32 parameters with block scales and nearest rounding)"""
    if param_update != "auto":
        return param_update
    plain = p_dtype_s == "float32" and variance_scale == "group" and round_type == "real-nearest"
    return "exact" if plain else "folded"


def traffic_source(rec):
    """where roofline.traffic comes from, in words"""
    if not rec:
        return "no counter record for these kernel sources"
    src = f"profiles/hbm_traffic.json, kernel sources {rec['source_hash']}"
    for half, counter in (("fetch", "FETCH_SIZE"), ("write", "WRITE_SIZE")):
        h = rec.get(f"{half}_source_hash", rec["source_hash"])
        if h != rec["source_hash"]:
            src += f"; the {counter} session ran on sources {h}"
    for k in ("write_note", "note"):
        if rec.get(k):
            src += f" ({rec[k]})"
    return src


def roofline_entry(m, workload, variance_scale, round_type, ceiling_gbs=None, param_update="auto"):
    from quantfour_adamw_cuda_amd import hbm_traffic
    achieved = m["algo_bytes"] / m["kernel_s"] / 1e9
    n = m["launches_per_step"]
    rec = hbm_traffic.lookup(workload, variance_scale, round_type, param_update)
    r = {
        "bound": "hbm",
        "kernel": "fused_4bit_kernel" if not m["rank1"] else "rank1_stats_kernel + fused_4bit_rank1_rows_kernel",
        "achieved": achieved,
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": achieved / HBM_PEAK_GBS,
        # per launch, averaged over the step's launches (they differ in size): HBM bytes from
        # hardware counters, algorithmic bytes, duration; achieved = algorithmic bytes / duration
        "traffic": rec["bytes_per_step"] / n if rec else None,
        "traffic_source": traffic_source(rec),
        "algorithmic_bytes_per_launch": m["algo_bytes"] / n,
        "kernel_ms_per_launch": m["kernel_s"] * 1e3 / n,
        "kernel_launches_per_step": n,
        "algorithmic_bytes_per_step": m["algo_bytes"],
        "kernel_ms_per_step": m["kernel_s"] * 1e3,
    }
    if ceiling_gbs:
        r["frac_of_ceiling"] = achieved / ceiling_gbs
    return r


def config_entry(name, desc, m, workload, variance_scale, round_type, p_dtype_s, g_dtype_s, param_update="auto"):
    r = roofline_entry(m, workload, variance_scale, round_type, param_update=param_update)
    return {
        "name": name,
        "workload": desc,
        "param_dtype": p_dtype_s,
        "grad_dtype": g_dtype_s,
        "variance_scale": variance_scale,
        "param_update": update_form_of(param_update, p_dtype_s, variance_scale, round_type),
        "steps": m["steps"],
        "ms_per_step": m["ms_per_step"],
        "params_per_s": m["total_params"] * m["steps"] / m["elapsed"],
        "host_ms_per_step": m["host_ms_per_step"],
        "kernel_ms_per_step": r["kernel_ms_per_step"],
        "kernel_launches_per_step": r["kernel_launches_per_step"],
        "algorithmic_bytes_per_step": r["algorithmic_bytes_per_step"],
        "achieved": r["achieved"],
        "frac": r["frac"],
        "traffic": r["traffic"],
    }


def load_probe():
    path = os.path.join(ROOT, "quantfour_adamw_cuda_amd", "csrc", "libq4probe.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it with `python -m quantfour_adamw_cuda_amd.build`")
    L = ctypes.CDLL(path)
    vp, u64, i = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int
    L.q4probe_copy.argtypes = [vp, vp, u64, vp]
    L.q4probe_read.argtypes = [vp, u64, vp, vp]
    L.q4probe_step_streams.argtypes = [vp, vp, vp, vp, vp, vp, u64, i, i, i, vp]
    for f in (L.q4probe_copy, L.q4probe_read, L.q4probe_step_streams):
        f.restype = i
    return L


def measure_ceiling(torch, device, reps=20):
    """Best of `reps` launches (after 3 untimed ones) of each probe on 2^30 elements, events on
    the launch stream around every launch.  The best, not the median: the figure stands for
    what the memory system can give such a kernel, and the step is compared with it."""
    L = load_probe()
    n = 1 << 30
    stream = torch.cuda.current_stream(device).cuda_stream
    tag = {"float32": 0, "bfloat16": 1}
    a = torch.empty(n, dtype=torch.float32, device=device).normal_()
    b = torch.empty(n, dtype=torch.float32, device=device).normal_()
    m = torch.zeros(n // 2, dtype=torch.uint8, device=device)
    v = torch.zeros(n // 2, dtype=torch.uint8, device=device)
    sm = torch.zeros(n // 128, dtype=torch.float32, device=device)
    sv = torch.zeros(n // 128, dtype=torch.float32, device=device)
    sink = torch.zeros(1, dtype=torch.int32, device=device)

    def timed(fn, mean=False):
        for _ in range(3):
            assert fn() == 0, "probe launch failed"
        torch.cuda.synchronize()
        evs = []
        for _ in range(reps):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            assert fn() == 0, "probe launch failed"
            e.record()
            evs.append((s, e))
        torch.cuda.synchronize()
        ms = [s.elapsed_time(e) for s, e in evs]
        return (sum(ms) / len(ms) if mean else min(ms)) / 1e3

    # the probes follow configurations of small kernels: bring the clocks back up first
    for _ in range(40):
        assert L.q4probe_copy(b.data_ptr(), a.data_ptr(), 4 * n, stream) == 0, "probe launch failed"
    torch.cuda.synchronize()

    out = {"unit": "GB/s", "elements": n, "launches": reps, "statistic": "best",
           "kernels": "libq4probe.so: probe_move_kernel (copy, read), probe_step_streams_kernel"}
    t = timed(lambda: L.q4probe_copy(b.data_ptr(), a.data_ptr(), 4 * n, stream))
    out["copy"] = 8.0 * n / t / 1e9
    t = timed(lambda: L.q4probe_read(a.data_ptr(), 4 * n, sink.data_ptr(), stream))
    out["read"] = 4.0 * n / t / 1e9
    def streams(p_s, g_s, which):
        return timed(lambda: L.q4probe_step_streams(a.data_ptr(), b.data_ptr(), m.data_ptr(), v.data_ptr(),
                                                    sm.data_ptr(), sv.data_ptr(), n, tag[p_s], tag[g_s], which, stream))

    for p_s, g_s in (("float32", "bfloat16"), ("float32", "float32"), ("bfloat16", "bfloat16"), ("bfloat16", "float32")):
        out[f"step_streams_{p_s}_{g_s}"] = n * bytes_per_param(p_s, g_s) / streams(p_s, g_s, 3) / 1e9
    # the headline's dtypes without the small streams: parameters read and written plus the
    # gradients read (10 bytes per element), and with the scales but not the codes (10.125)
    out["step_streams_float32_bfloat16_without_codes_and_scales"] = n * 10.0 / streams("float32", "bfloat16", 0) / 1e9
    out["step_streams_float32_bfloat16_without_codes"] = n * 10.125 / streams("float32", "bfloat16", 2) / 1e9
    # the same streams on 2^24 elements, the size of BASELINE.json configs[0]: what a launch of
    # that size can reach at all (ramp-up and drain are part of it)
    small = 1 << 24
    reps = 50
    t = timed(lambda: L.q4probe_step_streams(a.data_ptr(), b.data_ptr(), m.data_ptr(), v.data_ptr(), sm.data_ptr(),
                                             sv.data_ptr(), small, tag["float32"], tag["float32"], 3, stream))
    out["step_streams_float32_float32_2p24_elements"] = small * bytes_per_param("float32", "float32") / t / 1e9
    # and as the mean over the launches, the statistic the step's own figure is (its kernel time
    # is an average over the timed steps): at 40 us a launch the best and the mean lie 2-5 % apart
    t = timed(lambda: L.q4probe_step_streams(a.data_ptr(), b.data_ptr(), m.data_ptr(), v.data_ptr(), sm.data_ptr(),
                                             sv.data_ptr(), small, tag["float32"], tag["float32"], 3, stream), mean=True)
    out["step_streams_float32_float32_2p24_elements_mean"] = small * bytes_per_param("float32", "float32") / t / 1e9
    return out


def calibrate_copy(torch, device):
    """Three plain copies of 4 GiB (libq4probe.so), so that a counter profile of this command
    also holds a kernel whose traffic is known."""
    L = load_probe()
    src = torch.empty(1 << 30, dtype=torch.float32, device=device).normal_()
    dst = torch.empty_like(src)
    stream = torch.cuda.current_stream(device).cuda_stream
    for _ in range(3):
        assert L.q4probe_copy(dst.data_ptr(), src.data_ptr(), 4 << 30, stream) == 0
    torch.cuda.synchronize()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="llama3-8b", choices=sorted(WORKLOADS))
    ap.add_argument("--param-dtype", choices=DTYPE_NAMES, default=None, help="override the workload's parameter dtype")
    ap.add_argument("--grad-dtype", choices=DTYPE_NAMES, default=None, help="override the workload's gradient dtype")
    ap.add_argument("--grad-sets", type=int, default=2,
                    help="distinct pre-generated gradient sets rotated over the steps")
    ap.add_argument("--clip", choices=["none", "fused", "separate"], default="none",
                    help="also unscale the gradients by 1/1024 and clip them to a global norm of 1.0 "
                         "in every step: 'fused' = norm kernel + multiplier inside the step, "
                         "'separate' = torch's foreach multiply and clip_grad_norm_ passes, then the step")
    ap.add_argument("--variance-scale", choices=["group", "rank1"], default="group",
                    help="scaling of the second moment: per-128 block maxima (the fused CUDA path) or "
                         "rank-1 row/column maxima for matrices (a statistics pass precedes the update)")
    ap.add_argument("--round-type", choices=["real-nearest", "stochastic"], default="real-nearest",
                    help="rounding of the quantizer (stochastic: hash noise per element)")
    ap.add_argument("--param-update", choices=["auto", "exact", "folded"], default="auto",
                    help="form of the parameter update: exact = every operation of the reference's expression "
                         "rounded as IEEE 754 rounds it (bit-identical parameters), folded = hardware square root "
                         "and reciprocal (a tolerance), auto = exact for fp32 parameters with block scales and "
                         "nearest rounding, folded elsewhere")
    ap.add_argument("--configs", choices=["auto", "all", "none"], default="auto",
                    help="also time the other benchmark configurations and the step's variants and report "
                         "them in `configs` (auto: only for the default workload without variant options)")
    ap.add_argument("--no-ceiling", action="store_true", help="skip the memory-system probes")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--progress", action="store_true",
                    help="name every phase on stderr as it ends (stdout keeps its one JSON line), so that a "
                         "run that stops under a profiler shows where")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="for counter profiles: after the timed region, run the probe library's plain 4 GiB "
                         "copy three times, so that the profile also holds a kernel of known traffic, and run "
                         "W + K steps and no others (no host-time burst)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures the optimizer step on ONE GPU; the step needs "
                 "no collectives and every rank of a sharded job would run this same kernel "
                 "on its own shard. Run with --gpus 1.")

    import torch

    def phase(what):
        if args.progress:
            print(f"[bench] {what}", file=sys.stderr, flush=True)

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    shapes_fn, p_dtype_s, g_dtype_s, dist, desc = WORKLOADS[args.workload]
    p_dtype_s, g_dtype_s = args.param_dtype or p_dtype_s, args.grad_dtype or g_dtype_s
    plain = (args.variance_scale == "group" and args.round_type == "real-nearest" and args.clip == "none"
             and not args.param_dtype and not args.grad_dtype and args.param_update == "auto")
    all_configs = args.configs == "all" or (args.configs == "auto" and args.workload == "llama3-8b" and plain)

    params, grad_sets = build_inputs(torch, device, shapes_fn(), getattr(torch, p_dtype_s),
                                     getattr(torch, g_dtype_s), dist, args.grad_sets)
    phase(f"inputs of {args.workload} built")
    m = run_config(torch, params, grad_sets, p_dtype_s, g_dtype_s, args.steps, args.warmup,
                   args.variance_scale, args.round_type, args.clip, host_burst=not args.calibrate_copy,
                   param_update=args.param_update)
    phase("headline steps timed")
    if args.calibrate_copy:
        calibrate_copy(torch, device)
        phase("calibration copies done")

    out = {
        "metric": "params_updated_per_sec_fused_4bit_adamw_step",
        "value": m["total_params"] * args.steps / m["elapsed"],
        "unit": "params/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": m["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": desc,
            "tensors": len(params),
            "params": m["total_params"],
            "params_quantized": m["quant_params"],
            "param_dtype": p_dtype_s,
            "grad_dtype": g_dtype_s,
            "grad_sets": len(grad_sets),
            "param_update": update_form_of(args.param_update, p_dtype_s, args.variance_scale, args.round_type),
            "hyper": {"lr": HP["lr"], "betas": list(HP["betas"]), "eps": HP["eps"],
                      "weight_decay": HP["weight_decay"]},
        },
        "host_ms_per_step": m["host_ms_per_step"],
    }
    if args.round_type == "stochastic":
        out["config"]["workload"] += "; stochastic rounding"
    if m["rank1"]:
        out["config"]["workload"] += f"; rank-1 scaled second moment on {m['rank1']} matrices"
    if args.clip != "none":
        out["config"]["workload"] += f"; gradients unscaled by 1/1024 and clipped to norm 1.0 ({args.clip})"
        if "norm_s" in m:
            g_bytes = sum(g.numel() * g.element_size() for g in grad_sets[0])
            out["grad_norm"] = {"bound": "hbm", "kernel": "grad_sumsq_kernel", "ms_per_step": m["norm_s"] * 1e3,
                                "algorithmic_bytes_per_step": g_bytes, "achieved": g_bytes / m["norm_s"] / 1e9,
                                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": g_bytes / m["norm_s"] / 1e9 / HBM_PEAK_GBS}
    cpu = None if args.no_cpu_baseline else cpu_baseline(torch, params, grad_sets[0], HP)

    configs = []
    if all_configs:
        # the step's variants on the headline workload's own tensors, then the other configurations
        k, w = 10, 3
        for vs, rt, pu, name in (("group", "real-nearest", "folded", "folded parameter update (a tolerance instead of bit-identical parameters)"),
                                 ("group", "stochastic", "auto", "stochastic rounding"),
                                 ("rank1", "real-nearest", "auto", "rank-1 scaled second moment"),
                                 ("rank1", "stochastic", "auto", "rank-1 scaled second moment + stochastic rounding")):
            mv = run_config(torch, params, grad_sets, p_dtype_s, g_dtype_s, k, w, vs, rt, param_update=pu)
            configs.append(config_entry(f"{args.workload}, {name.split(' (')[0]}", desc + "; " + name, mv, args.workload, vs, rt,
                                        p_dtype_s, g_dtype_s, pu))
            phase(f"variant timed: {name}")
    del params, grad_sets
    torch.cuda.empty_cache()
    if all_configs:
        for wl, k, w in (("llama2-13b", 10, 3), ("gpt2-small", 200, 20), ("single-4096", 500, 50)):
            fn, ps, gs_, dist_, desc_ = WORKLOADS[wl]
            pr, gr = build_inputs(torch, device, fn(), getattr(torch, ps), getattr(torch, gs_), dist_, 2)
            mv = run_config(torch, pr, gr, ps, gs_, k, w)
            configs.append(config_entry(wl, desc_, mv, wl, "group", "real-nearest", ps, gs_))
            phase(f"configuration timed: {wl}")
            if wl == "llama2-13b":      # the 16-bit kernels' variants, the ones closest to the vector ALU's limit
                for vs, rt, pu, name in (("group", "real-nearest", "exact", "exact parameter update"),
                                         ("group", "stochastic", "auto", "stochastic rounding"),
                                         ("rank1", "real-nearest", "auto", "rank-1 scaled second moment")):
                    mv = run_config(torch, pr, gr, ps, gs_, k, w, vs, rt, param_update=pu)
                    configs.append(config_entry(f"{wl}, {name}", desc_ + "; " + name, mv, wl, vs, rt, ps, gs_, pu))
                    phase(f"variant timed: {wl}, {name}")
            del pr, gr
            torch.cuda.empty_cache()

    ceiling = None if args.no_ceiling else measure_ceiling(torch, device)
    phase("probes done")
    key = f"step_streams_{p_dtype_s}_{g_dtype_s}"
    out["roofline"] = roofline_entry(m, args.workload, args.variance_scale, args.round_type,
                                     ceiling.get(key) if ceiling else None, args.param_update)
    for c in configs:
        # block-scaled variants move the bytes of the probe with their element types; rank-1
        # scaling adds a second pass and the statistics, which no probe moves
        probe = ceiling.get(f"step_streams_{c['param_dtype']}_{c['grad_dtype']}") if ceiling else None
        c["frac_of_ceiling"] = c["achieved"] / probe if probe and c["variance_scale"] == "group" else None
        if ceiling and c["name"] == "single-4096":
            c["frac_of_ceiling_at_size"] = c["achieved"] / ceiling["step_streams_float32_float32_2p24_elements"]
            c["frac_of_ceiling_at_size_mean"] = c["achieved"] / ceiling["step_streams_float32_float32_2p24_elements_mean"]
    if cpu is not None:
        out["cpu_baseline"] = cpu
    if configs:
        out["configs"] = configs
    if ceiling is not None:
        out["ceiling"] = ceiling
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
