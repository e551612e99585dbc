"""AdamWFused_QuantFour: the host-side optimizer of the fused 4-bit AdamW step.

Mirrors the reference's optim/fused_quantfour.py:25-313 (class name, constructor
arguments and validation messages, `step()`, state keys) with the intended
behaviour where the reference's draft is unfinished:

  * moments are packed, two 4-bit codes per byte: uint8[(numel+1)//2]
    (the reference allocates numel bytes "for now", fused_quantfour.py:183)
  * block scales live in state[...]["overhead"]["max1"] and persist across steps
    (the reference re-creates them every step and swaps the two when passing them
    on, fused_quantfour.py:199-204, :274-275)
  * tensors of at most `param_quant_threshold` (4096) elements keep fp32 moments
    and take the non-quantized kernel (rule: optim/adamw_fourbit_triton.py:131-134;
    the reference forces the threshold to 2 and has no such branch,
    fused_quantfour.py:49, :180)
  * all tensors of a param group go to the device in one launch per kind instead
    of one launch plus one device synchronisation per tensor
    (fused_quantfour.py:171-292)

Beyond the reference's `step(closure)`: keyword arguments fold what its callers do
to the gradients between backward and step (tests/driver.py:53-59) into the step's
single read of them -- a multiplier (loss-scale removal), global-norm clipping, an
overflow flag that skips the step, and zeroing.  torch.amp.GradScaler.step() drives
the same path through the `grad_scale` / `found_inf` attributes it sets.

The step itself runs only in the HIP library (csrc/libq4adamw.so); without it,
or with parameters that are not on a GPU, `step()` raises.
"""
from itertools import chain, compress
from operator import attrgetter, is_, methodcaller
from typing import Any, Dict, Optional

import warnings

import numpy as np
import torch

from . import _lib
from . import quantfour_hip as _q

__all__ = ["AdamWFused_QuantFour", "enable_param_quantization"]


def enable_param_quantization(p, threshold) -> bool:
    """only enable quantization if the parameter is large enough
    (optim/fused_quantfour.py:18-22)"""
    if threshold and p.numel() <= threshold:
        return False
    return True


class _Bucket:
    """One launch of a step: the tensors of one (kind, device, dtypes, step) and their
    descriptor array."""
    __slots__ = ("kind", "device", "idx", "arr", "p_tag", "g_tag", "salts", "g_dtypes", "g_column")


class _Plan:
    """A param group's launches and what they rest on (see _build_plan / _refresh_plan)."""
    __slots__ = ("gi", "capturable", "stochastic", "state_obj", "params_obj", "param_ids", "all_params",
                 "has_grad", "plannable", "params", "p_ptrs", "step_views", "grads", "buckets", "held")


class AdamWFused_QuantFour(torch.optim.Optimizer):
    """Fused 4bit AdamW for MI355X"""

    def __init__(
        self,
        params,
        lr=1e-3,
        betas=(0.9, 0.999),
        eps=1e-8,
        weight_decay=1e-2,
        *,
        fused: Optional[bool] = False,
        variance_scale_type: str = "group",
        round_type: str = "real-nearest",
        seed: Optional[int] = None,
        capturable: bool = False,
        param_update: str = "auto",
    ):
        # optim/fused_quantfour.py:38-47
        if not 0.0 < lr:
            raise ValueError(f"Invalid learning rate: {lr=}")
        if not 0.0 < eps:
            raise ValueError(f"Invalid eps value: {eps=}")
        if not 0.0 < betas[0] < 1.0:
            raise ValueError(f"Invalid Beta[0]: {betas[0]=}")
        if not 0.0 < betas[1] < 1.0:
            raise ValueError(f"Invalid Beta[1]: {betas[1]=}")
        if not 0.0 <= weight_decay:
            raise ValueError(f"Invalid weight_decay value: {weight_decay=}")

        # how the second moment is scaled before it is quantized: "group" = one abs-max per
        # 128 consecutive elements, what the fused CUDA path does (cuda_adamw_kernels.cu:353-383);
        # "rank1" = min(row maximum, column maximum) for matrices, the draft's SecondMoment
        # setting (adamw_fourbit_triton.py:124, :834-863), one statistic per dimension for
        # tensors of two to four dimensions of any sizes; 1-D tensors keep group scaling, as
        # there (:841-846), and so do tensors of five and more dimensions or with a last
        # dimension of 1
        if variance_scale_type not in ("group", "rank1"):
            raise ValueError(f"Invalid variance_scale_type: {variance_scale_type=}")
        self.variance_scale_type = variance_scale_type

        # rounding of the quantizer: "real-nearest" (the fused CUDA path and the draft's setting,
        # quant_opt_base.py:28) or "stochastic" (the quantize_bsearch<STOCHASTIC> rule the draft
        # quotes, adamw_fourbit_triton.py:1050-1075).  The noise seed is drawn once and, as in the
        # draft (adamw_fourbit_triton.py:163-165), agreed on across ranks; it travels in the
        # param groups, so a resumed run continues the same noise sequence.
        if round_type not in ("real-nearest", "stochastic"):
            raise ValueError(f"Invalid round_type: {round_type=}")
        if round_type == "stochastic" and seed is None:
            seed_t = torch.randint(1 << 31, size=[1])
            if torch.distributed.is_available() and torch.distributed.is_initialized():
                on_gpu = torch.distributed.get_backend() == "nccl"
                seed_t = seed_t.cuda() if on_gpu else seed_t
                torch.distributed.broadcast(seed_t, src=0)
                seed_t = seed_t.cpu()
            seed = int(seed_t)

        # capturable: the step number lives on the device (one counter per param group and
        # device), so that step() can be captured in a graph and every replay is the next
        # step; a tensor lr (one float32 on the parameters' device) is read by the kernels,
        # a float lr, betas, eps and weight_decay are fixed when the graph is captured.  As
        # for torch.optim.AdamW(capturable=True); the reference reads its step counter on the
        # host (optim/fused_quantfour.py:178, :286-290) and cannot be captured.

        # how the quantized step computes the parameter: "exact" = the reference's expression
        # (optim/cuda_adamw_kernels.cu:334,351) with each of its seven operations rounded as
        # IEEE 754 rounds it, so the parameters come out bit-identical to it; "folded" = the
        # short form with the hardware's square root and reciprocal (fp32 parameters within
        # 1e-6 of max(|p|, |step|), 16-bit ones within an ulp of their type); "auto" = exact
        # where it costs under 1 % of the step (fp32 parameters, block scales, nearest
        # rounding: the reference's own path), folded elsewhere (5 to 10 %)
        if param_update not in _lib.UPDATE_FORMS:
            raise ValueError(f"Invalid param_update: {param_update=}")

        # tensors with numel <= threshold are not quantized
        # (FirstMoment.threshold / SecondMoment.threshold, adamw_fourbit_triton.py:118, :128)
        self.param_quant_threshold = 4096

        defaults = dict(
            lr=lr,
            betas=betas,
            eps=eps,
            weight_decay=weight_decay,
            fused=fused,
            round_type=round_type,
            seed=seed,
            capturable=capturable,
            param_update=param_update,
        )
        super().__init__(params, defaults)
        self._launch_cache: Dict[Any, Any] = {}
        self._step_buffers: Dict[Any, Any] = {}
        self._device_steps: Dict[Any, Any] = {}
        self._plans: Dict[Any, Any] = {}
        self._warned_unaligned = False
        # global gradient norm of the last step(max_grad_norm=...), a device scalar
        self.last_grad_norm = None
        self._norm_buffers: Dict[Any, Any] = {}
        # set to a list to collect ("fused_4bit" | "fused_single_tensor" | "grad_norm", start, end)
        # event triples around every launch, recorded on the launch stream
        self.kernel_timing = None

    # -- state ------------------------------------------------------------
    def init_qstate(self, p, state_name):
        """optim/fused_quantfour.py:61-70"""
        state = self.state[p]
        field = f"{state_name}_qstate"
        state[field] = {
            "enable": True,
            "overhead": dict(),
            "qmap": None,
        }
        state[field]["enable"] = enable_param_quantization(p, self.param_quant_threshold)

    def __getstate__(self) -> Dict[str, Any]:
        """The base class pickles defaults, state and param groups; the settings that live
        on the object travel with them (launch caches and device counters do not)."""
        state = super().__getstate__()
        state["variance_scale_type"] = self.variance_scale_type
        state["param_quant_threshold"] = self.param_quant_threshold
        return state

    def __setstate__(self, state: Dict[str, Any]) -> None:
        """optim/fused_quantfour.py:73-84"""
        super().__setstate__(state)
        self._launch_cache = {}
        self._step_buffers = {}
        self._device_steps = {}
        self._plans = {}
        self._norm_buffers = {}
        self.__dict__.setdefault("kernel_timing", None)
        self.__dict__.setdefault("_warned_unaligned", False)
        self.__dict__.setdefault("last_grad_norm", None)
        self.__dict__.setdefault("variance_scale_type", "group")
        self.__dict__.setdefault("param_quant_threshold", 4096)
        self.__dict__.pop("_pending_skip", None)
        self.__dict__.pop("_skip_flag_host", None)
        for group in self.param_groups:
            group.setdefault("fused", None)
            group.setdefault("round_type", "real-nearest")
            group.setdefault("seed", None)
            group.setdefault("capturable", False)
            group.setdefault("param_update", "auto")
        state_values = list(self.state.values())
        step_is_tensor = len(state_values) != 0 and torch.is_tensor(state_values[0]["step"])
        if not step_is_tensor:
            for s in state_values:
                s["step"] = torch.tensor(float(s["step"]))

    def _init_state(self, p):
        """Lazy state of one parameter (optim/fused_quantfour.py:110-120, :180-204)."""
        state = self.state[p]
        state["step"] = torch.tensor(0.0)
        self.init_qstate(p, "momentum")
        self.init_qstate(p, "variance")
        if state["momentum_qstate"]["enable"]:
            nbytes, nblk = _q.state_sizes(p.numel())
            # zero codes with zero scales dequantize to m = -0.0 and v = 0
            state["exp_avg"] = torch.zeros((nbytes,), dtype=torch.uint8, device=p.device)
            state["exp_avg_sq"] = torch.zeros((nbytes,), dtype=torch.uint8, device=p.device)
            state["momentum_qstate"]["overhead"]["max1"] = torch.zeros(
                (nblk,), dtype=torch.float32, device=p.device)
            if self._use_rank1(p):
                self._init_rank1_overhead(p, state["variance_qstate"]["overhead"])
            else:
                state["variance_qstate"]["overhead"]["max1"] = torch.zeros(
                    (nblk,), dtype=torch.float32, device=p.device)
        else:
            state["exp_avg"] = torch.zeros_like(p, dtype=torch.float32,
                                                memory_format=torch.contiguous_format)
            state["exp_avg_sq"] = torch.zeros_like(p, dtype=torch.float32,
                                                   memory_format=torch.contiguous_format)

    def _param_position(self, p):
        """Index of p among all parameters of all groups (stable across runs and resumes)."""
        pos = self.__dict__.get("_positions")
        if pos is None or p not in pos:
            pos = {q_: i for i, q_ in enumerate(chain.from_iterable(g["params"] for g in self.param_groups))}
            self._positions = pos
        return pos[p]

    def _use_rank1(self, p):
        return self.variance_scale_type == "rank1" and _q.rank1_eligible(p)

    @staticmethod
    def _init_rank1_overhead(p, overhead, stats=None):
        """Statistics of a rank-1-scaled second moment, keys as in the draft's metadata
        (adamw_fourbit_triton.py:846-852): max_dims = one statistic per dimension in keepdim
        shape (for a matrix: row maxima [rows, 1], column maxima [1, cols]), max1 = None;
        scratch_dims are same-sized buffers the step accumulates the new maxima in (zeros
        between steps).  Tensors of more than two dimensions also keep the scale of every
        flattened row, the minimum over its leading statistics (derived; row_scale), and a
        scratch of that size.  stats: the statistics to start from, one per dimension."""
        z = lambda *shape: torch.zeros(shape, dtype=torch.float32, device=p.device)
        keep = [[p.shape[d] if d == j else 1 for d in range(p.dim())] for j in range(p.dim())]
        overhead["dim"] = p.dim()
        overhead["max1"] = None
        overhead["max_dims"] = [z(*keep[j]) if stats is None else
                                stats[j].detach().to(device=p.device, dtype=torch.float32, copy=True).reshape(keep[j])
                                for j in range(p.dim())]
        overhead["scratch_dims"] = [z(*keep[j]) for j in range(p.dim())]
        if p.dim() > 2:
            lead = [t.reshape(-1) for t in overhead["max_dims"][:-1]]
            overhead["row_scale"] = _q.rank1_row_scale(lead, p.shape[:-1])
            overhead["row_scratch"] = z(overhead["row_scale"].numel())

    @staticmethod
    def _rank1_buffers(p, overhead):
        """(rows' statistic or scale, last dimension's statistic, their scratch buffers,
        leading statistics or None) as the rank-1 entry points take them."""
        dims, scratch = overhead["max_dims"], overhead["scratch_dims"]
        if p.dim() == 2:
            return dims[0], dims[1], scratch[0], scratch[1], None
        return (overhead["row_scale"], dims[-1], overhead["row_scratch"], scratch[-1],
                ([t.view(-1) for t in dims[:-1]], [t.view(-1) for t in scratch[:-1]]))

    def _init_group(
        self,
        group,
        params_with_grad,
        grads,
        exp_avgs,
        exp_avgs_sqs,
        state_steps,
        momentum_meta,
        variance_meta,
        momentum_quant_enabled,
    ):
        """optim/fused_quantfour.py:87-128"""
        for p in group["params"]:
            if p.grad is None:
                continue
            if p.grad.is_sparse:
                raise RuntimeError("QuantFour AdamW does not support sparse gradients")
            if p.numel() == 0:
                continue
            grads.append(p.grad)
            params_with_grad.append(p)
            state = self.state[p]
            if len(state) == 0:
                self._init_state(p)
            state_steps.append(state["step"])
            exp_avgs.append(state["exp_avg"])
            exp_avgs_sqs.append(state["exp_avg_sq"])
            momentum_meta.append(state["momentum_qstate"]["overhead"])
            variance_meta.append(state["variance_qstate"]["overhead"])
            momentum_quant_enabled.append(state["momentum_qstate"]["enable"])

    def load_state_dict(self, state_dict):
        """Accepts this optimizer's own state_dict and, as a migration path, the state_dict
        of torch.optim.AdamW (fp32 `exp_avg` / `exp_avg_sq` shaped like the parameter):
        moments of tensors above the quantization threshold are quantized on load
        (per-128 abs-max scaling, nearest code), the others are kept in fp32."""
        super().load_state_dict(state_dict)
        # The base class casts every state tensor to the parameter's dtype.  Packed codes
        # are uint8, block scales and non-quantized moments fp32, whatever the parameter
        # is: take them from the source again, keeping their dtype.
        saved_ids = chain.from_iterable(g["params"] for g in state_dict["param_groups"])
        own = chain.from_iterable(g["params"] for g in self.param_groups)
        for pid, p in zip(saved_ids, own):
            src = state_dict["state"].get(pid)
            if src is None:
                continue
            dst = self.state[p]
            if torch.is_tensor(dst.get("step")):
                # the base class hands the source's own tensor on; step() advances it in place
                dst["step"] = dst["step"].detach().clone()
            for key in ("exp_avg", "exp_avg_sq"):
                if torch.is_tensor(src.get(key)):
                    dst[key] = src[key].detach().to(device=p.device, copy=True)
            for key in ("momentum_qstate", "variance_qstate"):
                overhead = src.get(key, {}).get("overhead", {})
                max1 = overhead.get("max1")
                if torch.is_tensor(max1):
                    dst[key]["overhead"]["max1"] = max1.detach().to(
                        device=p.device, dtype=torch.float32, copy=True)
                if "max_dims" in overhead:      # rank-1 statistics; scratch and derived row scales are made anew
                    self._init_rank1_overhead(p, dst[key]["overhead"], overhead["max_dims"])
            if "momentum_qstate" not in src:
                self._adopt_adamw_state(p, dst)
        self._launch_cache = {}
        self._plans = {}
        self._device_steps = {}      # device step counters restart from the loaded host numbers

    def _adopt_adamw_state(self, p, state):
        """Turns one parameter's torch.optim.AdamW state (step, exp_avg, exp_avg_sq in the
        parameter's shape) into this optimizer's layout (optim/fused_quantfour.py:65-70,
        :112-119, :199-204)."""
        if "max_exp_avg_sq" in state:
            raise ValueError("amsgrad state (max_exp_avg_sq) cannot be taken over")
        if not torch.is_tensor(state["step"]):
            state["step"] = torch.tensor(float(state["step"]))
        state["step"] = state["step"].detach().to(device="cpu", dtype=torch.float32).reshape(())
        exp_avg = state["exp_avg"].detach().to(device=p.device, dtype=torch.float32)
        exp_avg_sq = state["exp_avg_sq"].detach().to(device=p.device, dtype=torch.float32)
        if exp_avg.numel() != p.numel() or exp_avg_sq.numel() != p.numel():
            raise ValueError("AdamW state does not match the parameter's size")
        self.init_qstate(p, "momentum")
        self.init_qstate(p, "variance")
        if state["momentum_qstate"]["enable"]:
            state["exp_avg"], state["momentum_qstate"]["overhead"]["max1"] = _q.quantize_state(exp_avg, 0)
            if self._use_rank1(p) and p.dim() == 2:
                codes, rmax, cmax = _q.quantize_state_rank1(exp_avg_sq.reshape(p.shape))
                state["exp_avg_sq"] = codes
                self._init_rank1_overhead(p, state["variance_qstate"]["overhead"], [rmax, cmax])
            elif self._use_rank1(p):
                # one statistic per dimension (maximum over all others); the rows of the tensor
                # flattened to [rows, last dimension] are scaled by the minimum over their
                # leading statistics (adamw_fourbit_triton.py:738-755)
                v = torch.nan_to_num(exp_avg_sq.reshape(p.shape).abs(), nan=0.0, posinf=float("inf"))
                stats = [v.amax(dim=[d for d in range(p.dim()) if d != j]) for j in range(p.dim())]
                overhead = state["variance_qstate"]["overhead"]
                self._init_rank1_overhead(p, overhead, stats)
                state["exp_avg_sq"] = _q.quantize_state_rank1_scaled(
                    exp_avg_sq.reshape(-1, p.shape[-1]), overhead["row_scale"], overhead["max_dims"][-1].view(-1))
            else:
                state["exp_avg_sq"], state["variance_qstate"]["overhead"]["max1"] = _q.quantize_state(exp_avg_sq, 1)
        else:
            state["exp_avg"] = exp_avg.contiguous().clone()
            state["exp_avg_sq"] = exp_avg_sq.contiguous().clone()

    def adamw_state_dict(self):
        """This optimizer's state in the layout of torch.optim.AdamW: fp32 moments shaped
        like their parameter (quantized moments are dequantized: code-book entry times
        block scale).  `torch.optim.AdamW(params).load_state_dict(opt.adamw_state_dict())`
        continues training in full precision."""
        sd = self.state_dict()
        own = list(chain.from_iterable(g["params"] for g in self.param_groups))
        ids = list(chain.from_iterable(g["params"] for g in sd["param_groups"]))
        out_state = {}
        for pid, p in zip(ids, own):
            st = self.state.get(p)
            if not st:
                continue
            if st["momentum_qstate"]["enable"]:
                m = _q.dequantize_state(st["exp_avg"], st["momentum_qstate"]["overhead"]["max1"], p.numel(), 0)
                v_meta = st["variance_qstate"]["overhead"]
                if "max_dims" in v_meta:
                    rmax, cmax = self._rank1_buffers(p, v_meta)[:2]
                    v = _q.dequantize_state_rank1(st["exp_avg_sq"], rmax.reshape(-1), cmax.reshape(-1))
                else:
                    v = _q.dequantize_state(st["exp_avg_sq"], v_meta["max1"], p.numel(), 1)
            else:
                m, v = st["exp_avg"].clone(), st["exp_avg_sq"].clone()
            out_state[pid] = {"step": st["step"].detach().clone(),
                              "exp_avg": m.view(p.shape), "exp_avg_sq": v.view(p.shape)}
        groups = []
        for g in sd["param_groups"]:
            groups.append({"lr": g["lr"], "betas": g["betas"], "eps": g["eps"],
                           "weight_decay": g["weight_decay"], "amsgrad": False, "maximize": False,
                           "foreach": None, "capturable": False, "differentiable": False,
                           "fused": None, "params": list(g["params"])})
        return {"state": out_state, "param_groups": groups}

    # -- step -------------------------------------------------------------
    # torch.amp.GradScaler.step() hands its scale and overflow flag to an optimizer that
    # declares this, as attributes `grad_scale` and `found_inf`, instead of unscaling
    # the gradients in a pass of its own
    _step_supports_amp_scaling = True

    def _grad_multiplier(self, grad_scale, max_grad_norm):
        """(host float, device float32 scalar or None): the factor every gradient is
        multiplied by inside the step."""
        host, dev = 1.0, None
        if torch.is_tensor(grad_scale):
            dev = grad_scale.detach().to(torch.float32).reshape(1)
        elif grad_scale is not None:
            host = float(grad_scale)
        amp_scale = getattr(self, "grad_scale", None)   # set by GradScaler: divide by it
        if amp_scale is not None:
            inv = amp_scale.detach().double().reciprocal().float().reshape(1)
            dev = inv if dev is None else dev * inv
        if max_grad_norm is None:
            return host, dev
        # global norm of the multiplied gradients, per dtype on the device, combined there
        by_dtype: Dict[Any, list] = {}
        for group in self.param_groups:
            for p in group["params"]:
                if p.grad is not None:
                    by_dtype.setdefault((p.grad.device, p.grad.dtype), []).append(p.grad)
        if not by_dtype:
            return host, dev
        devices = {d for d, _ in by_dtype}
        assert len(devices) == 1, "max_grad_norm needs all gradients on one device"
        device = devices.pop()
        outs = []
        for key, gs in by_dtype.items():
            bufs = self._norm_buffers.get(key)
            if bufs is None:
                bufs = (torch.empty(3, dtype=torch.float32, device=device),
                        torch.empty(_lib.NORM_WORKSPACE_BYTES // 8, dtype=torch.float64, device=device))
                self._norm_buffers[key] = bufs
            if self.kernel_timing is None:
                outs.append(_q.grad_norm(gs, host, dev, float(max_grad_norm), out=bufs[0], workspace=bufs[1]))
            else:
                with torch.cuda.device(device):
                    start = torch.cuda.Event(enable_timing=True)
                    end = torch.cuda.Event(enable_timing=True)
                    start.record()
                    outs.append(_q.grad_norm(gs, host, dev, float(max_grad_norm), out=bufs[0], workspace=bufs[1]))
                    end.record()
                self.kernel_timing.append(("grad_norm", start, end))
        if len(outs) == 1:
            self.last_grad_norm = outs[0][0]
            return 1.0, outs[0][2:3]
        total = torch.linalg.vector_norm(torch.stack([o[0] for o in outs]))
        coef = torch.clamp(float(max_grad_norm) / (total + 1e-6), max=1.0)
        self.last_grad_norm = total
        mult = coef * host if dev is None else coef * host * dev
        return 1.0, mult.reshape(1)

    @torch.no_grad()
    def step(self, closure=None, *, grad_scale=None, found_inf=None, max_grad_norm=None,
             zero_grad=False):
        """single optimization step

        grad_scale     number or one-element tensor: every gradient is multiplied by it
                       inside the step (e.g. 1 / loss scale); the stored gradients stay
                       as they are
        max_grad_norm  clip the (multiplied) gradients to this global L2 norm, as
                       torch.nn.utils.clip_grad_norm_ would, without rewriting them;
                       the norm is left in `last_grad_norm` (a device scalar)
        found_inf      one-element float32 device tensor: a non-zero value makes the
                       device leave parameters and state alone (gradients are still
                       cleared if zero_grad asks for it), without synchronising; the step
                       counters of a skipped step are taken back when the next step
                       (or state_dict()) looks at the flag's value, which by then has
                       reached the host
        zero_grad      overwrite the gradients with zeros once the step has read them,
                       or once an overflow flag has cancelled it
        """
        loss = None
        if closure:
            with torch.enable_grad():
                loss = closure()

        self._settle_skipped_step()
        if found_inf is None:
            found_inf = getattr(self, "found_inf", None)    # set by GradScaler
        if found_inf is not None:
            found_inf = found_inf.detach().to(torch.float32).reshape(1)
        host_mult, dev_mult = self._grad_multiplier(grad_scale, max_grad_norm)
        stepped = []   # step counters advanced by this call

        _lib.load()  # raises if the HIP library has not been built

        # everything is gathered and validated before the first launch and before any step
        # counter moves, so that a refusal leaves parameters, state and counters as they were
        ready = []
        for gi, group in enumerate(self.param_groups):
            plan = self._plans.get(gi)
            if plan is None or not self._refresh_plan(group, plan):
                plan = self._build_plan(gi, group)
            if plan is not None:
                ready.append((group, plan))
        for group, plan in ready:
            self._run_plan(group, plan, host_mult, dev_mult, found_inf, zero_grad, stepped)

        if found_inf is not None and stepped:
            self._watch_skip_flag(found_inf, stepped)
        return loss

    def _build_plan(self, gi, group):
        """One param group's launches from scratch: gathers the parameters that have a gradient
        and their state (created on first use), sorts them into launch buckets -- one per
        (kind, device, dtypes, step) -- and validates everything.  The plan it returns (None:
        no parameter has a gradient) is kept, so that the following steps only have to check
        that nothing it rests on has changed (_refresh_plan).  Replaces the per-parameter
        loop of optim/fused_quantfour.py:171-292."""
        params_with_grad = []
        grads = []
        exp_avgs = []
        exp_avg_sqs = []
        state_steps = []
        momentum_meta = []
        variance_meta = []
        momentum_quant_enabled = []

        self._init_group(
            group,
            params_with_grad,
            grads,
            exp_avgs,
            exp_avg_sqs,
            state_steps,
            momentum_meta,
            variance_meta,
            momentum_quant_enabled,
        )
        self._plans.pop(gi, None)
        if not params_with_grad:
            return None

        capturable = bool(group.get("capturable", False))
        stochastic = group.get("round_type", "real-nearest") == "stochastic"
        if capturable and len(params_with_grad) != sum(1 for p in group["params"] if p.numel() > 0):
            raise ValueError("capturable=True needs a gradient for every parameter of the group: "
                             "the group's parameters share one step counter on the device")
        self._layout_steps(gi, params_with_grad, state_steps)
        steps_now = self._step_buffers[gi][0].tolist()

        buckets: Dict[Any, list] = {}
        for i, param in enumerate(params_with_grad):
            assert param.is_cuda, "param must be on cuda"
            kind = momentum_quant_enabled[i]
            if kind and "max_dims" in variance_meta[i]:
                kind = "rank1_sr" if stochastic else "rank1"
            elif kind and stochastic:
                kind = "sr"
            key = (kind, param.device, param.dtype, grads[i].dtype, 0.0 if capturable else steps_now[i])
            buckets.setdefault(key, []).append(i)

        plan = _Plan()
        plan.gi = gi
        plan.capturable = capturable
        plan.stochastic = stochastic
        plan.state_obj = self.state
        plan.params_obj = group["params"]
        plan.param_ids = list(map(id, group["params"]))
        plan.all_params = tuple(group["params"])          # keeps the ids above from being reused
        plan.has_grad = [p.grad is not None for p in group["params"]]
        plan.plannable = all(p.numel() > 0 for p in group["params"])
        plan.params = params_with_grad
        plan.p_ptrs = [t.data_ptr() for t in params_with_grad]
        if not self._warned_unaligned and any(ptr % 16 for ptr, t in zip(plan.p_ptrs, params_with_grad)
                                              if t.numel() > self.param_quant_threshold):
            # legal (the kernels' 16-byte accesses need the element type's alignment only) but
            # slower: neighbouring waves' stores then share lines
            self._warned_unaligned = True
            warnings.warn("AdamWFused_QuantFour: a quantized parameter does not start on a 16-byte boundary "
                          "(a view into a flat buffer?); its step takes 6 to 9 % longer than an aligned one's",
                          stacklevel=3)
        plan.step_views = state_steps
        plan.grads = grads
        plan.buckets = []
        for (quantized, device, p_dtype, g_dtype, _), idx in buckets.items():
            cached = self._bucket_table(
                (gi, quantized, device, p_dtype, g_dtype),
                [params_with_grad[i] for i in idx], [grads[i] for i in idx], [exp_avgs[i] for i in idx],
                [exp_avg_sqs[i] for i in idx], [momentum_meta[i] for i in idx], [variance_meta[i] for i in idx])
            _, arr, (p_tag, g_tag, *extra) = cached
            b = _Bucket()
            b.kind, b.device, b.idx, b.arr, b.p_tag, b.g_tag = quantized, device, idx, arr, p_tag, g_tag
            b.salts = extra[0] if extra else None
            b.g_dtypes = [g_dtype] * len(idx)
            # the gradient pointers inside the descriptor array: the second 8-byte field of
            # every descriptor type (include/q4adamw.h)
            b.g_column = np.frombuffer(arr, dtype=np.uint64).reshape(len(idx), -1)[:, 1]
            plan.buckets.append(b)
        # what the plan rests on besides the parameters: the state tensors, by identity.
        # core: (state dict, step, exp_avg, exp_avg_sq) per parameter; extra: (dict, key,
        # tensor or list) for the scales and statistics of the quantized ones
        core, extra = [], []
        for i, param in enumerate(params_with_grad):
            core.append((self.state[param], state_steps[i], exp_avgs[i], exp_avg_sqs[i]))
            if momentum_quant_enabled[i]:
                extra.append((momentum_meta[i], "max1", momentum_meta[i]["max1"]))
                for key in ("max1", "max_dims", "scratch_dims", "row_scale", "row_scratch"):
                    if key in variance_meta[i]:
                        extra.append((variance_meta[i], key, variance_meta[i][key]))
        held = (core, extra)
        plan.held = held
        if plan.plannable:
            self._plans[gi] = plan
        return plan

    def _refresh_plan(self, group, plan):
        """True if the plan of the last step still describes this group -- the same parameters
        at the same addresses, the same ones with a gradient, the same state tensors, dense
        contiguous gradients of the same dtypes -- after pointing its descriptors at this
        step's gradients.  False sends the group through _build_plan, which also words the
        refusals."""
        params = group["params"]
        if (params is not plan.params_obj or self.state is not plan.state_obj
                or bool(group.get("capturable", False)) != plan.capturable
                or (group.get("round_type", "real-nearest") == "stochastic") != plan.stochastic
                or list(map(id, params)) != plan.param_ids):
            return False
        all_grads = list(map(attrgetter("grad"), params))
        if [g is not None for g in all_grads] != plan.has_grad:
            return False
        grads = list(compress(all_grads, plan.has_grad))
        if list(map(methodcaller("data_ptr"), plan.params)) != plan.p_ptrs:
            return False
        core, extra = plan.held
        try:
            for st, step, exp_avg, exp_avg_sq in core:
                if st["step"] is not step or st["exp_avg"] is not exp_avg or st["exp_avg_sq"] is not exp_avg_sq:
                    return False
            for holder, key, held in extra:
                if holder[key] is not held:
                    return False
        except KeyError:
            return False
        steps_now = self._step_buffers[plan.gi][0].tolist()
        pointers = []
        # a gradient object that was validated last step still has its dtype, size and device;
        # its strides are looked at again (t_() or as_strided_() re-stride a tensor in place,
        # and the kernels would read it as if it were dense), and its address is read again
        seen = all(map(is_, grads, plan.grads))
        for b in plan.buckets:
            gs = [grads[i] for i in b.idx]
            # is_contiguous() is False for a sparse tensor
            if not all(map(methodcaller("is_contiguous"), gs)):
                return False
            if not seen:
                if list(map(attrgetter("dtype"), gs)) != b.g_dtypes:
                    return False
                for g, i in zip(gs, b.idx):
                    p = plan.params[i]
                    if g.numel() != p.numel() or g.device != p.device:
                        return False
            ptrs = np.fromiter(map(methodcaller("data_ptr"), gs), dtype=np.uint64, count=len(gs))
            if not plan.capturable and len({steps_now[i] for i in b.idx}) != 1:
                return False
            pointers.append(ptrs)
        for b, ptrs in zip(plan.buckets, pointers):
            b.g_column[:] = ptrs
        plan.grads = grads
        return True

    def _run_plan(self, group, plan, host_mult, dev_mult, found_inf, zero_grad, stepped):
        """Advances the step counters of the plan's parameters (optim/fused_quantfour.py:178)
        and makes one launch per bucket."""
        gi, capturable = plan.gi, plan.capturable
        beta1, beta2 = group["betas"]
        # a tensor lr is read on the device in capturable mode; otherwise its value is taken now
        lr = 1.0 if capturable else float(group["lr"])
        weight_decay = group["weight_decay"]
        eps = group["eps"]
        before = ([float(s) for s in plan.step_views]
                  if capturable and not self._has_device_steps(gi) else None)
        steps = self._advance_steps(gi, plan.params, plan.step_views)
        if not capturable:       # a capturable group's true counter is on the device
            stepped.extend(plan.step_views)
        step_consts = {}
        if capturable:
            # one counter per device: advance it and derive the step's scalars there
            for device in {b.device for b in plan.buckets}:
                step_consts[device] = self._device_step(gi, device, group, before, found_inf)
        for b in plan.buckets:
            rank1 = b.kind in ("rank1", "rank1_sr")
            # lr and step of a capturable group enter through step_consts; the arguments only
            # pass the range check
            t_step = 1.0 if capturable else steps[b.idx[0]]
            options = _q.grad_options(b.device, host_mult, dev_mult, found_inf, zero_grad,
                                      step_consts.get(b.device), group.get("param_update", "auto"))
            hyper = (b.device, b.p_tag, b.g_tag, beta1, beta2, lr, weight_decay, eps, t_step, options)
            if b.kind in ("sr", "rank1_sr"):
                launch = _q.launch_rank1_table_sr if rank1 else _q.launch_table_sr
                args = (b.arr, b.salts, group["seed"]) + hyper
            else:
                launch = (_q.launch_rank1_table if rank1 else
                          _q.launch_table if b.kind else _q.launch_small_table)
                args = (b.arr,) + hyper
            if self.kernel_timing is None:
                launch(*args)
            else:
                with _q._on(b.device):
                    start = torch.cuda.Event(enable_timing=True)
                    end = torch.cuda.Event(enable_timing=True)
                    start.record()
                    launch(*args)
                    end.record()
                kind = ("fused_4bit_rank1" if rank1 else
                        "fused_4bit" if b.kind else "fused_single_tensor")   # stochastic rounding counts as its scaling's kind
                self.kernel_timing.append((kind, start, end))

    # -- capturable: the step number on the device ------------------------------------
    def _has_device_steps(self, gi):
        return any(k[0] == gi for k in self._device_steps)

    def _device_step(self, gi, device, group, steps_before, found_inf):
        """Advances the device step counter of (param group, device) and returns the buffer
        that holds the new step's derived scalars.  The counter starts from the host's
        number of steps taken, which all parameters of the group must share."""
        beta1, beta2 = group["betas"]
        key = (gi, device)
        st = self._device_steps.get(key)
        if st is None:
            if steps_before is None:     # another device of this group exists already: same number
                other = next(v for k, v in self._device_steps.items() if k[0] == gi)
                first = float(other["counter"])
            else:
                if len(set(steps_before)) != 1:
                    raise ValueError("capturable=True needs all parameters of a group at the same step")
                first = steps_before[0]
            st = dict(counter=torch.full((1,), first, dtype=torch.float32, device=device),
                      table=_q.make_bias_table(float(beta1), float(beta2), device),
                      consts=_q.new_step_consts(device), betas=(float(beta1), float(beta2)),
                      lr_dev=None, lr_host=None)
            self._device_steps[key] = st
        if st["betas"] != (float(beta1), float(beta2)):
            st["table"] = _q.make_bias_table(float(beta1), float(beta2), device)
            st["betas"] = (float(beta1), float(beta2))
        lr = group["lr"]
        if torch.is_tensor(lr):
            assert lr.is_cuda and lr.device == device and lr.dtype == torch.float32 and lr.numel() == 1, \
                "a tensor lr must be one float32 on the parameters' device"
            lr_dev, lr_host = lr.reshape(1), 1.0
        else:
            if st["lr_dev"] is None:
                st["lr_dev"] = torch.empty(1, dtype=torch.float32, device=device)
            if st["lr_host"] != float(lr):      # refreshed only when the host's value changes
                st["lr_dev"].fill_(float(lr))
                st["lr_host"] = float(lr)
            lr_dev, lr_host = st["lr_dev"], float(lr)
        _q.device_step(st["counter"], st["table"], st["consts"], float(beta1), float(beta2), lr_host,
                       group["weight_decay"], group["eps"], lr_dev=lr_dev, found_inf=found_inf)
        return st["consts"]

    def _sync_host_steps(self):
        """capturable: the device counters are the truth (replays of a captured graph do not
        pass through step()); copies them into the parameters' host step counters."""
        for (gi, device), st in self._device_steps.items():
            value = float(st["counter"])          # synchronises
            for p in self.param_groups[gi]["params"]:
                s = self.state.get(p)
                if s and p.device == device and torch.is_tensor(s.get("step")):
                    s["step"].fill_(value)

    def _bucket_table(self, cache_key, ps, gs, ms, vs, m_meta, v_meta):
        """(pointers, ctypes descriptor array, (param tag, grad tag[, salts])) of one launch
        bucket.  Parameters and state stay where they are from step to step; gradients usually
        do not: the array is rebuilt (and everything validated) only when a parameter or state
        pointer changed, otherwise the gradients' pointers are refreshed in place."""
        _, quantized, device, _, _ = cache_key
        rank1 = quantized in ("rank1", "rank1_sr")
        if rank1:
            sms = [mm["max1"] for mm in m_meta]
            bufs = [self._rank1_buffers(p, vm) for p, vm in zip(ps, v_meta)]
            stats = [[b[d] for b in bufs] for d in range(4)]   # rows, last dimension, their scratch
            leads = [b[4] for b in bufs]
            fixed = (ps, ms, vs, sms, *stats, [t for ld in leads if ld is not None for ts in ld for t in ts])
        elif quantized:
            sms = [mm["max1"] for mm in m_meta]
            svs = [vm["max1"] for vm in v_meta]
            fixed = (ps, ms, vs, sms, svs)
        else:
            fixed = (ps, ms, vs)
        ptrs = tuple(t.data_ptr() for ts in fixed for t in ts)
        cached = self._launch_cache.get(cache_key)
        if cached is None or cached[0] != ptrs:
            if rank1:
                arr = _q.make_rank1_table(ps, gs, ms, vs, sms, stats[0], stats[1], stats[2], stats[3], leads)
            elif quantized:
                arr = _q.make_table(ps, gs, ms, vs, sms, svs)
            else:
                arr = _q.make_small_table(ps, gs, ms, vs)
            tags = (_q._tag(ps[0], "param"), _q._tag(gs[0], "grad"))
            if quantized in ("sr", "rank1_sr"):   # noise salt of a tensor: its position among all parameters
                tags += (_q.make_salts([self._param_position(p) for p in ps]),)
            cached = (ptrs, arr, tags)
            self._launch_cache[cache_key] = cached
        else:
            arr = cached[1]
            for i, (p, g) in enumerate(zip(ps, gs)):
                # dtype and device are part of the bucket key (optim/fused_quantfour.py:255-261)
                assert g.device == device, "grad must be on the param's device"
                assert g.is_contiguous(), "grad must be contiguous"
                assert g.numel() == p.numel(), f"grad numel {g.numel()} != param numel {p.numel()}"
                arr[i].g = g.data_ptr()
        return cached

    def _layout_steps(self, gi, params, state_steps):
        """Makes the step counters of `params` 0-dim views of one host buffer (values kept)
        and `state_steps` the list of those views, unless they are already."""
        cached = self._step_buffers.get(gi)
        if (cached is None or len(cached[1]) != len(state_steps)
                or not all(map(is_, cached[1], state_steps))):
            buf = torch.stack([t.detach().to(device="cpu", dtype=torch.float32).reshape(())
                               for t in state_steps])
            views = list(buf.unbind(0))
            for p, v in zip(params, views):
                self.state[p]["step"] = v
            cached = (buf, views)
            self._step_buffers[gi] = cached
            state_steps[:] = views
        return cached[0]

    def _advance_steps(self, gi, params, state_steps):
        """Adds 1 to every step counter and returns their new values as Python floats.  The
        counters of a group's parameters are 0-dim views of one host buffer, so this is one
        addition whatever the number of tensors; a counter that was replaced (lazy state,
        load_state_dict, the user) is noticed by identity and the buffer is laid out again.
        `state_steps` is updated in place to the tensors the state holds afterwards."""
        buf = self._layout_steps(gi, params, state_steps)
        buf.add_(1)
        return buf.tolist()

    # -- overflow flag: keeping the step counters right without a synchronisation -----
    def _watch_skip_flag(self, found_inf, stepped):
        """Starts an asynchronous copy of the flag to pinned host memory; an event marks its
        arrival.  The next step() or state_dict() reads it."""
        host = self.__dict__.get("_skip_flag_host")
        if host is None:
            host = torch.empty(1, dtype=torch.float32, pin_memory=True)
            self._skip_flag_host = host
        with torch.cuda.device(found_inf.device):
            host.copy_(found_inf, non_blocking=True)
            arrived = torch.cuda.Event()
            arrived.record()
        self._pending_skip = (arrived, stepped)

    def _settle_skipped_step(self):
        """If the previous step ran under an overflow flag that turned out set, the device did
        nothing: take its advance of the step counters back.  Waits for that step's flag
        only (it has long arrived when the next step begins)."""
        pending = self.__dict__.pop("_pending_skip", None)
        if pending is None:
            return
        arrived, stepped = pending
        arrived.synchronize()
        if float(self._skip_flag_host[0]) != 0.0:
            torch._foreach_sub_(stepped, 1)

    def state_dict(self):
        self._settle_skipped_step()
        self._sync_host_steps()
        return super().state_dict()
