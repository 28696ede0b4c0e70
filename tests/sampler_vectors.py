"""Sampler cases in which the order of the reference's operations decides the token
(`src/sampling/sampler.zig:56-79,186-201`); each names the token the reference's order gives
and what a plausible other order would give.  Run through the plain sampler, the product's host
sampler and the device sampler."""
import math

# (logits, history, parameters, uniform numbers to try, token that must come out, why)
ORDER_CASES = [
    # repetition divides first, then presence is taken off: 4/2 - 1 = 1.0 < 1.2; presence first
    # would give (4 - 1)/2 = 1.5 > 1.2
    ([4.0, 1.2], [0], dict(temperature=0.0, repetition_penalty=2.0, presence_penalty=1.0),
     [0.5], 1, "repetition before presence"),
    # 4/2 - 3 * 0.3 = 1.1 < 1.2; frequency first would give (4 - 0.9)/2 = 1.55
    ([4.0, 1.2], [0, 0, 0], dict(temperature=0.0, repetition_penalty=2.0, frequency_penalty=0.3),
     [0.5], 1, "repetition before frequency, frequency times the count"),
    # a negative logit is multiplied: -1 * 2 = -2 < -1.9; divided it would be -0.5
    ([-1.0, -1.9], [0], dict(temperature=0.0, repetition_penalty=2.0),
     [0.5], 1, "a negative logit is multiplied by the repetition penalty"),
    # tokens that were not seen keep their logits whatever the penalties are
    ([1.0, 1.1], [], dict(temperature=0.0, repetition_penalty=5.0, presence_penalty=9.0),
     [0.5], 1, "penalties touch seen tokens only"),
    # exp(l - max) = [1, 0.6, 0.4].  min-p 0.5 keeps [1, 0.6] (sum 1.6); top-p 0.6 on the
    # renormalised kept set: 1/1.6 = 0.625 >= 0.6 keeps one candidate, so token 0 whatever
    # u is.  Without the renormalisation (1/2 = 0.5 < 0.6), or with top-p before min-p, two
    # candidates stay and u = 0.9 draws token 1.
    ([math.log(5.0), math.log(3.0), math.log(2.0)], [],
     dict(temperature=1.0, top_k=3, min_p=0.5, top_p=0.6),
     [0.0, 0.3, 0.63, 0.9, 0.999], 0, "top-p after min-p, on the renormalised kept set"),
    # the same numbers without min-p: top-p 0.6 keeps two (0.5 < 0.6 <= 0.8), so u = 0.9
    # (0.9 * 1.6 = 1.44 > 1) draws token 1 and u = 0.3 token 0: the cut above is min-p's doing
    ([math.log(5.0), math.log(3.0), math.log(2.0)], [],
     dict(temperature=1.0, top_k=3, top_p=0.6), [0.9], 1, "top-p keeps the candidate that crosses"),
    ([math.log(5.0), math.log(3.0), math.log(2.0)], [],
     dict(temperature=1.0, top_k=3, top_p=0.6), [0.3], 0, "the walk starts at the best"),
    # temperature divides before the exponential: at T = 0.5 the ratios square, [1, .36, .16],
    # min-p 0.3 keeps [1, .36]; at T = 1 it would keep all three.  u = 0.99 then draws token 1,
    # not token 2
    ([math.log(5.0), math.log(3.0), math.log(2.0)], [],
     dict(temperature=0.5, top_k=3, min_p=0.3), [0.99], 1, "temperature before min-p"),
]


class FixedU:
    """A random stream that always gives the same uniform number."""

    def __init__(self, u):
        self.u = u

    def float64(self):
        return self.u
