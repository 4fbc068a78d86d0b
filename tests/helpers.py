"""Comparison helpers shared by the parity tests."""
import torch

# tolerances of the parity bar: rtol = atol per dtype for outputs, plus scale-aware bounds that stay
# meaningful when the output magnitude is far below atol (routed-expert outputs are ~1e-3)
OUT_TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 2e-2}
FRO_TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 2e-3}


def rel_fro(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float(((a - b).norm() / b.norm().clamp_min(1e-300)).item())


def max_rel_to_scale(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-300))


def assert_output_close(got, ref, dtype, what=""):
    """The stated bar (allclose with rtol = atol per dtype) and the scale-aware bars."""
    tol = OUT_TOL[dtype]
    g, r = got.float().cpu(), ref.float().cpu()
    assert g.shape == r.shape, f"{what}: shape {g.shape} vs {r.shape}"
    assert torch.isfinite(g).all(), f"{what}: non-finite values"
    torch.testing.assert_close(g, r, rtol=tol, atol=tol, msg=lambda m: f"{what}: {m}")
    fro, mx = rel_fro(g, r), max_rel_to_scale(g, r)
    assert fro <= FRO_TOL[dtype], f"{what}: relative Frobenius error {fro:.3e} > {FRO_TOL[dtype]:.1e}"
    assert mx <= 2 * tol, f"{what}: max|diff|/max|ref| = {mx:.3e} > {2 * tol:.1e}"


def cuda(*ts):
    out = tuple(None if t is None else t.cuda() for t in ts)
    return out if len(out) > 1 else out[0]


def assert_mostly_close(got, ref, dtype, what="", max_outliers=1e-4):
    """Against an oracle evaluated in a 16-bit dtype: that oracle rounds every intermediate (gate, up,
    their product, each partial output) to 16 bits, so its own noise reaches the tolerance in the far
    tail when rows are long.  All but a 1e-4 fraction of the elements must meet rtol = atol, and the
    scale-aware bounds must hold for the whole tensor."""
    tol = OUT_TOL[dtype]
    g, r = got.detach().float().cpu(), ref.detach().float().cpu()
    bad = ((g - r).abs() > tol + tol * r.abs()).float().mean().item()
    assert bad <= max_outliers, f"{what}: {bad:.2e} of the elements outside rtol=atol={tol}"
    assert rel_fro(g, r) <= FRO_TOL[dtype], f"{what}: relative Frobenius error {rel_fro(g, r):.3e}"
    assert max_rel_to_scale(g, r) <= 2 * tol, f"{what}: max|diff|/max|ref| = {max_rel_to_scale(g, r):.3e}"
    return bad
