"""Shared test helpers: seeded inputs and the error metrics of the parity bar."""
import numpy as np
import torch

# Parity bar for attention outputs and gradients (bf16 in, bf16 out, fp32 oracle):
#   max abs error  <= 2e-2 * max(s, |ref|) per element, with s = min(1, max|ref| over the tensor):
#       absolute (2e-2) for tensors of N(0,1) scale, relative to |ref| above 1 (dK/dV sum over heads
#       and rows and reach magnitudes of 8..16, where one bf16 ulp is already 0.06), and for a tensor
#       whose values are small everywhere (outputs and gradients of rows that average hundreds of
#       thousands of keys: 1e-4..1e-2) relative to its own largest value, so that such a tensor is
#       held to a bound a wrong result fails rather than to one 500 times its values.
#   mean relative error <= 1e-3, where
#       mre(x, ref) = mean|x - ref| / mean|ref|
#   is taken in excess of the oracle's own bf16 representation error mre(bf16(ref), ref).
# The kernels return bf16, and rounding the exact fp32 result to bf16 already costs
# mre = 1.39e-3 on N(0,1) data (mean of ulp/4 over a binade), so 1e-3 on the raw figure is
# below what any bf16 output can reach; measured against the representable result the bar
# is meaningful: a dropped key, a wrong mask column or a wrong scale moves mre by 1e-2 or more.
MAX_ABS_TOL = 2e-2
MEAN_REL_TOL = 1e-3
ZERO_REF = 1e-6   # a reference whose largest value is below this is taken to be zero (inputs are of N(0,1) scale)


def randn_bf16(shape, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float32).to(torch.bfloat16)


def make_qkv(total_q, total_k, hq, hkv, d, seed):
    q = randn_bf16((total_q, hq, d), 1000 + seed)
    k = randn_bf16((total_k, hkv, d), 2000 + seed)
    v = randn_bf16((total_k, hkv, d), 3000 + seed)
    do = randn_bf16((total_q, hq, d), 4000 + seed)
    return q, k, v, do


def mre(x: torch.Tensor, ref: torch.Tensor) -> float:
    return ((x - ref).abs().mean() / ref.abs().mean().clamp_min(1e-30)).item()


def errors(got: torch.Tensor, ref: torch.Tensor):
    """(max abs error, mean relative error in excess of the bf16 rounding floor of ref)."""
    e = error_figures(got, ref)
    return e["max_abs_scaled"], e["mre_excess"]


def error_figures(got: torch.Tensor, ref: torch.Tensor) -> dict:
    """Every figure the parity bar is stated in, raw and as asserted:
      max_abs        max |x - ref|                              (raw)
      mre            mean|x - ref| / mean|ref|                  (raw)
      floor          mre(round(ref), ref): what rounding the exact result to the output type (bf16; fp16 for fp16 outputs) costs
      max_abs_scaled max |x - ref| / max(s, |ref|), s = min(1, max|ref|)   (asserted <= 2e-2)
      mre_excess     mre - floor                                (asserted <= 1e-3)
      ref_absmax     max |ref|"""
    out_dtype = got.dtype if got.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    diff = (got - ref).abs()
    floor = mre(ref.to(out_dtype).float(), ref)   # what rounding the exact result to the kernel's output type costs
    raw = mre(got, ref)
    ref_absmax = ref.abs().max().item()
    scale = max(min(1.0, ref_absmax), 1e-30)
    return dict(max_abs=diff.max().item(), mre=raw, floor=floor, max_abs_scaled=(diff / ref.abs().clamp_min(scale)).max().item(),
                mre_excess=raw - floor, ref_absmax=ref_absmax, numel=ref.numel())


# Every comparison made through assert_close_bf16 in this process: (test id, tensor, figures).  The session hook in
# conftest.py writes them out so that the raw figures behind the asserted ones can be read from a run's records.
PARITY_LOG = []


def assert_close_bf16(got, ref, what, max_abs=MAX_ABS_TOL, mean_rel=MEAN_REL_TOL):
    assert tuple(got.shape) == tuple(ref.shape), f"{what}: shape {tuple(got.shape)} against {tuple(ref.shape)}"
    if ref.numel() == 0:
        return 0.0, 0.0
    assert torch.isfinite(got.float()).all(), f"{what}: non-finite values"
    e = error_figures(got, ref)
    ma, mr = e["max_abs_scaled"], e["mre_excess"]
    import os
    PARITY_LOG.append((os.environ.get("PYTEST_CURRENT_TEST", "").split(" ")[0], what, e))
    print(f"    parity {what}: raw max|x-ref| {e['max_abs']:.3e} (max|ref| {e['ref_absmax']:.2f}), raw mean-rel {e['mre']:.3e} "
          f"(bf16 floor of ref {e['floor']:.3e}); asserted {ma:.3e} <= {max_abs}, {mr:.3e} <= {mean_rel}", flush=True)
    if e["ref_absmax"] <= ZERO_REF:
        # a reference that is zero up to fp32 rounding noise (dQ / dK of a one-token document: its single probability
        # is 1 whatever the score): relative figures mean nothing, the result must be zero to the same degree
        got_absmax = got.detach().float().abs().max().item()
        assert got_absmax <= 10 * ZERO_REF, f"{what}: reference is zero (max {e['ref_absmax']:.1e}), result reaches {got_absmax:.3e}"
        return 0.0, 0.0
    assert ma <= max_abs and mr <= mean_rel, (
        f"{what}: max abs {ma:.3e} (tol {max_abs}), mean rel above bf16 floor {mr:.3e} (tol {mean_rel}); "
        f"raw max abs {e['max_abs']:.3e}, raw mean rel {e['mre']:.3e}")
    return ma, mr


def cu(lens):
    return np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)


def task_sums(a, b, cu, hkv, chunk=32768):
    """(sum of a*b, sum of (a*b)^2) per (task, kv head) in fp64; query heads fold onto their kv head.
    Tokens are processed in chunks so that the fp64 temporaries of a 524288-token batch stay small."""
    t, h, d = a.shape
    parts = []
    for s0 in range(0, t, chunk):
        prod = a[s0:s0 + chunk].double() * b[s0:s0 + chunk].double()
        n = prod.shape[0]
        parts.append(torch.stack([prod.sum(2), (prod * prod).sum(2)], 0).reshape(2, n, hkv, h // hkv).sum(3))   # [2, n, hkv]
    per_tok = torch.cat(parts, 1) if parts else torch.zeros(2, 0, hkv, dtype=torch.float64, device=a.device)
    csum = torch.cat([torch.zeros_like(per_tok[:, :1]), per_tok.cumsum(1)], 1)
    idx = torch.as_tensor(np.asarray(cu), device=a.device, dtype=torch.long)
    seg = csum[:, idx[1:]] - csum[:, idx[:-1]]
    return seg[0].cpu(), seg[1].cpu()


def assert_identity(lhs, rhs, what):
    """Both sides are sums of products of bf16-rounded kernel outputs with exact inputs: every
    product carries an independent relative error of up to 2^-8 (output rounding, plus the bf16
    rounding of P and dS ahead of the MFMAs), so the sums agree to a few standard deviations of
    2^-8 * sqrt(sum of squared products).  8 sigma allowed."""
    (a, a2), (b, b2) = lhs, rhs
    tol = 8 * 2.0 ** -8 * torch.sqrt(a2 + b2) + 1e-6
    bad = (a - b).abs() > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} (task, kv head) cells off, worst {((a - b).abs() / tol).max().item():.1f} x tol"
