"""What the GPU tests compare the engine's logits with, and how closely.

float32: the plain implementation's logits, at float32 tolerances.

bfloat16: the yardstick is the reference's own arithmetic in that type.  The plain implementation is run
twice: in float32 (the exact logits) and with the roundings of the reference's bfloat16 run
(plain_llama.forward(..., rounding="reference")).  The distance of the second from the first, position by
position, is what bfloat16 costs the reference.  Two bounds follow from it:
  * at every position the engine's error is at most MARGIN times the reference's error there, or MARGIN
    times the reference's typical error over the sequence (its 90th percentile) where the reference
    happened to be lucky: rounding errors are random, and at single positions the ratio of two draws has a
    long tail.  Measured over every check of this folder (four tiny configurations and two layers of the
    8B and 7B shapes): the engine is at most 1.72 times that far, so MARGIN is 2.5; where attention is
    made sharp (test_far_key_decides) rounding is amplified unevenly and the worst position is 2.12 times
    that far, so SHARP_MARGIN is 3.  A lost key moves those logits by their whole scale, ten times the bound;
  * over 32 positions or more the engine's mean error is at most MEAN_MARGIN times the reference's.  The
    engine rounds in fewer places (float32 residual stream, one rounding per norm, float32 logits) and
    must not be the worse of the two: measured, its mean error is 0.70 to 0.98 of the reference's.
A key lost at a page border or a slot read from another sequence moves a position's logits by a multiple of
what rounding does.
"""

import torch

import plain_llama as P

MARGIN = 2.5
SHARP_MARGIN = 3.0
MEAN_MARGIN = 1.25


class Expected:
    """Exact logits [..., vocab]; for bfloat16 also the reference's own error at each position [...] and its
    typical error over the sequence the position belongs to [...]."""

    def __init__(self, logits: torch.Tensor, ref_error=None, typical=None):
        self.logits, self.ref_error, self.typical = logits, ref_error, typical

    @property
    def shape(self):
        return self.logits.shape

    def __getitem__(self, index):
        if self.ref_error is None:
            return Expected(self.logits[index])
        return Expected(self.logits[index], self.ref_error[index], self.typical[index])

    @staticmethod
    def _join(items, how):
        if items[0].ref_error is None:
            return Expected(how([i.logits for i in items]))
        return Expected(how([i.logits for i in items]), how([i.ref_error for i in items]), how([i.typical for i in items]))

    @staticmethod
    def stack(items):
        return Expected._join(items, torch.stack)

    @staticmethod
    def cat(items):
        return Expected._join(items, torch.cat)


def expect(weights, cfg, ids, dtype, **how) -> Expected:
    """how: further arguments of the plain forward (calls=...: the sequence as it was fed, for ntk scaling)."""
    exact = P.forward(weights, cfg, ids, **how)
    if dtype in ("float32", torch.float32):
        return Expected(exact)
    reference = P.forward(weights, cfg, ids, storage=torch.bfloat16, rounding="reference", **how)
    error = (reference - exact).abs().amax(dim=-1)
    return Expected(exact, error, torch.quantile(error, 0.9).expand_as(error))


def check(got, want, dtype, margin: float = MARGIN) -> None:
    got = got.float().cpu()
    if not isinstance(want, Expected):
        want = Expected(want)
    assert got.shape == want.shape, f"{tuple(got.shape)} logits, {tuple(want.shape)} expected"
    if dtype in ("float32", torch.float32):
        torch.testing.assert_close(got, want.logits, atol=2e-4, rtol=1e-3)
        return
    assert want.ref_error is not None, "bfloat16 logits are judged against the reference's bfloat16 error"
    error = (got - want.logits).abs().amax(dim=-1).flatten()
    ref, typical = want.ref_error.flatten(), want.typical.flatten()
    allowed = margin * torch.maximum(ref, typical)
    worst = int(torch.argmax(error / allowed))
    assert bool((error <= allowed).all()), (
        f"bfloat16 logits are {float(error[worst]):.4g} off at row {worst}; the reference's own bfloat16 arithmetic is "
        f"{float(ref[worst]):.4g} off there and typically {float(typical[worst]):.4g} (allowed: {margin} times the larger)")
    if error.numel() >= 32:
        assert float(error.mean()) <= MEAN_MARGIN * float(ref.mean()), (
            f"bfloat16 logits are {float(error.mean()):.4g} off on average, the reference's own arithmetic {float(ref.mean()):.4g}")
