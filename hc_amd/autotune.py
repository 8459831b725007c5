"""`autotune(kernel, *args)`: choose tunable values and kernel variants by timing.

The reference specifies this flow in docs/langref.md:471-586 (TunableParam,
`tunables=` on the decorator, `autotune(kernel, args...)` returning parameters
that `kernel.parametrize(...)` accepts, and `save` / `autotune.load`); it ships
no implementation.  Here a kernel body is bound to a hand-written kernel that
re-tiles the work for the hardware, so two things can be tuned:

  * the kernel's own TunableParam symbols.  They change which windows the body
    covers per group and therefore whether and how it binds; combinations that
    do not bind are skipped.
  * the variant of the hand-written kernel family the body binds to (vector
    width, rows per workgroup, tile shape, ...: hcamdSetVariant).

Every candidate is run on the arguments given, so pass arrays that may be
overwritten (a reduction accumulates into its result cell on every trial).
"""

from __future__ import annotations

import itertools
import json
import math

from . import runtime as rt
from .binding import NoNativeKernel
from .indexing import sym

# C entry point -> (variant family, variant numbers worth trying)
_FAMILIES = {
    "hcamdLaunchAddF32": ("add", tuple(range(1, 9))),
    "hcamdLaunchFmaF16": ("fma", tuple(range(1, 7))),
    "hcamdLaunchCopy2D": ("copy", tuple(range(1, 9))),
    "hcamdLaunchSoftmaxF32": ("softmax", (0, 3, 4, 5, 6, 7, 8, 9, 10, 11)),
    "hcamdLaunchQuantizeF16I8": ("quantize", (0, 2, 3, 4, 7, 8, 9, 10, 11)),
    "hcamdLaunchGemmBF16": ("gemm", (1, 2, 3, 4, 5, 7, 8, 9, 10, 11, 12)),
    "hcamdGatherGemmLaunchF32": ("gather", (1, 2, 3, 4, 5, 6)),
    "hcamdGatherGemmLaunch": ("gather", (1, 2, 3, 4)),
}


class TunedParams(dict):
    """{symbol: value} for kernel.parametrize(), plus `variants`
    ({family: number}) and the device they were measured on."""

    def __init__(self, symbols=(), variants=None, device="", microseconds=None):
        super().__init__(symbols)
        self.variants = dict(variants or {})
        self.device = device
        self.microseconds = microseconds

    def save(self, path) -> None:
        with open(path, "w") as f:
            json.dump({"symbols": {str(k): int(v) for k, v in self.items()},
                       "variants": self.variants, "device": self.device,
                       "microseconds": self.microseconds}, f, indent=1)

    @staticmethod
    def load(path) -> "TunedParams":
        with open(path) as f:
            d = json.load(f)
        return TunedParams({getattr(sym, k): v for k, v in d["symbols"].items()},
                           d.get("variants"), d.get("device", ""), d.get("microseconds"))


def _time(plans, ctx, iters, warmup) -> float:
    for _ in range(warmup):
        for p in plans:
            p.launch()
    ctx.synchronize()
    start, stop = rt.Event(ctx), rt.Event(ctx)
    start.record()
    for _ in range(iters):
        for p in plans:
            p.launch()
    stop.record()
    ctx.synchronize()
    return start.elapsed_ms(stop) * 1e3 / iters


def _tunables(kernel):
    t = kernel.tunables
    return [t] if hasattr(t, "sym") else list(t)


def autotune(kernel, *args, max_trials: int = 64, iters: int = 10, warmup: int = 2,
             tune_variants: bool = True) -> TunedParams:
    """Times `kernel` on `args` over its tunables' values (all combinations if
    there are at most `max_trials`, otherwise one symbol at a time) and over the
    variants of the hand-written kernel it binds to; returns the fastest."""
    ctx = rt.default_context(kernel.device)
    tun = _tunables(kernel)
    best = {t.sym: t.default for t in tun}

    def measure(values):
        try:
            plans = kernel.parametrize(values).plan(*args, ctx=ctx)
        except (NoNativeKernel, RuntimeError, AssertionError):
            return math.inf, None
        try:
            return _time(plans, ctx, iters, warmup), plans
        except rt.HcRuntimeError:
            return math.inf, None

    best_us, best_plans = measure(best)
    spaces = [list(t.vals) for t in tun]
    if tun and math.prod(len(s) for s in spaces) <= max_trials:
        for combo in itertools.product(*spaces):
            cand = {t.sym: v for t, v in zip(tun, combo)}
            us, plans = measure(cand)
            if us < best_us:
                best, best_us, best_plans = cand, us, plans
    else:
        per_symbol = max(1, max_trials // max(len(tun), 1))
        for t, space in zip(tun, spaces):
            step = max(1, len(space) // per_symbol)
            for v in space[::step]:
                cand = {**best, t.sym: v}
                us, plans = measure(cand)
                if us < best_us:
                    best, best_us, best_plans = cand, us, plans
    if best_plans is None:
        raise NoNativeKernel("autotune: no combination of the tunables binds to a native kernel")

    variants = {}
    if tune_variants:
        for what in {p.what for p in best_plans}:
            if what not in _FAMILIES:
                continue
            family, numbers = _FAMILIES[what]
            chosen = 0
            # (this thread's choice only: whatever the process has selected with
            # hcamdSetVariant stays as it is, and is what other threads keep running)
            try:
                for v in numbers:
                    rt.set_thread_variant(family, v)
                    try:
                        us = _time(best_plans, ctx, iters, warmup)
                    except rt.HcRuntimeError:
                        continue
                    if us < best_us:
                        best_us, chosen = us, v
            finally:
                rt.set_thread_variant(family, -1)
            if chosen:
                variants[family] = chosen
    return TunedParams(best, variants, ctx.info().get("arch", ""), round(best_us, 3))


autotune.load = TunedParams.load
