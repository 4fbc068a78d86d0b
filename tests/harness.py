"""Benchmark + validation harness for reference-style throughput tests (`pytest -s` prints one table per case).

Same idea as the reference's tests/testing.py (a list of implementations labelled by backend, the first one is the
numerical baseline, each is timed over warm-up + repeats with peak-memory columns; tolerances per dtype as in
tests/testing.py:269-281), with one difference that matters: a mismatch against the baseline **fails** the test
instead of being printed.
"""
from __future__ import annotations

import dataclasses
import statistics
import time
from typing import Any, Callable, List, Sequence

import torch

BASELINE, HIP = "pytorch", "hip"
TOLERANCE = {torch.float32: 1e-2, torch.float16: 1e-1, torch.bfloat16: 1e-1}   # rtol = atol, tests/testing.py:269-281


@dataclasses.dataclass
class Impl:
    backend: str                      # "pytorch" (baseline, first in the list) or "hip"
    fn: Callable[..., Any]


@dataclasses.dataclass
class Result:
    backend: str
    dtype: torch.dtype
    times_ms: List[float]
    flops: float
    peak_alloc_mib: float
    peak_reserved_mib: float

    @property
    def mean_ms(self) -> float:
        return statistics.fmean(self.times_ms)

    @property
    def tflops(self) -> float:
        return self.flops / (self.mean_ms * 1e-3) / 1e12 if self.flops else 0.0


def tensors_of(out: Any) -> List[torch.Tensor]:
    if torch.is_tensor(out):
        return [out]
    if isinstance(out, (tuple, list)):
        return [t for item in out for t in tensors_of(item)]
    return []


def check_against(out: Any, ref: Any, what: str) -> None:
    """Every floating tensor of `out` within the dtype's tolerance of `ref`; integer tensors are compared by the caller."""
    outs, refs = tensors_of(out), tensors_of(ref)
    assert len(outs) == len(refs), f"{what}: {len(outs)} tensors vs {len(refs)} in the baseline"
    for i, (o, r) in enumerate(zip(outs, refs)):
        assert o.shape == r.shape, f"{what}[{i}]: shape {tuple(o.shape)} vs {tuple(r.shape)}"
        if o.is_floating_point():
            tol = TOLERANCE.get(r.dtype, 1e-5)
            torch.testing.assert_close(o.float(), r.float(), rtol=tol, atol=tol, msg=lambda m: f"{what}[{i}]: {m}")


def time_impl(impl: Impl, make_args: Callable[[], Sequence[Any]], flops: float, warmup: int, repeat: int) -> Result:
    out = None
    for _ in range(warmup):
        out = impl.fn(*make_args())
    torch.cuda.synchronize()
    times, alloc, reserved = [], 0, 0
    for _ in range(repeat):
        args = make_args()
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        t0 = time.perf_counter()
        out = impl.fn(*args)
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3)
        alloc, reserved = max(alloc, torch.cuda.max_memory_allocated()), max(reserved, torch.cuda.max_memory_reserved())
    first = tensors_of(out)
    return Result(impl.backend, first[0].dtype if first else torch.float32, times, flops, alloc / 2**20, reserved / 2**20)


def run(impls: Sequence[Impl], make_args: Callable[[], Sequence[Any]], *, flops: float, what: str, warmup: int = 3,
        repeat: int = 20, validate: Callable[[Any, Any], None] | None = None) -> List[Result]:
    """Validate every implementation against the first one on the same fresh inputs (assertion), then time them all."""
    base = impls[0].fn(*make_args())
    torch.cuda.synchronize()
    for impl in impls[1:]:
        out = impl.fn(*make_args())
        torch.cuda.synchronize()
        (validate or (lambda o, r: check_against(o, r, f"{what} ({impl.backend})")))(out, base)
    del base
    results = [time_impl(impl, make_args, flops, warmup, repeat) for impl in impls]
    show(results, what)
    return results


def show(results: Sequence[Result], what: str) -> None:
    print(f"\n[{what}]")
    print(f"{'backend':<10} {'dtype':>10} {'speed ms':>10} {'speedup':>10} {'tflops':>10} {'peak MiB':>10}")
    print("-" * 66)
    for r in results:
        print(f"{r.backend:<10} {str(r.dtype).replace('torch.', ''):>10} {r.mean_ms:>10.3f} {results[0].mean_ms / r.mean_ms:>10.2f} "
              f"{r.tflops:>10.3f} {r.peak_alloc_mib:>10.2f}")
