"""CPU restatement of the reference's token sampler -- TEST INFRASTRUCTURE ONLY (tests/ may
import it; nothing shipped does).

Follows sampler.cpp:18-101 and kernels/cpu/softmax.cpp:6-21 statement by statement in numpy
float32 (sequential sums are written as loops so that the rounding order is the reference's),
with std::minstd_rand0 restated as the Lehmer generator x <- 16807 x mod (2^31 - 1).

Pinned by the reference's own vectors in tests/test_sampler.cpp (greedy cases :37-74,
deterministic cuts :96-121, the seeded known answer :157-169) and by its statistical cases
(:76-95, :132-155); see tests/test_sampler.py.
"""
import numpy as np

F = np.float32


class MinStdRand0:
    """std::minstd_rand0: multiplier 16807, modulus 2^31-1, min 1, max 2^31-2."""
    M = 2147483647

    def __init__(self, seed=1):
        self.seed(seed)

    def seed(self, s):
        s = int(s) % self.M
        self.x = s if s != 0 else 1  # the standard maps a zero state to 1

    def __call__(self):
        self.x = (self.x * 16807) % self.M
        return self.x

    min = 1
    max = M - 1


def softmax(logits):
    """kernels/cpu/softmax.cpp:6-21 at temperature 1: fp32, sum in index order."""
    x = np.asarray(logits, F)
    e = np.exp((x - x.max()) / F(1.0)).astype(F)
    s = F(0)
    for v in e:
        s = F(s + v)
    return (e / s).astype(F)


def sample(logits, temperature, top_k, top_p, gen):
    """Sampler::Sample (sampler.cpp:38-99).  Ties between equal probabilities are ordered by
    index (std::sort leaves that order unspecified)."""
    temperature = F(min(max(F(temperature), F(0.1)), F(5.0)))
    probs = softmax(logits)
    order = sorted(range(len(probs)), key=lambda i: (-float(probs[i]), i))
    length = len(order)
    cumsum = F(0)
    for i, idx in enumerate(order):  # top-p
        cumsum = F(cumsum + probs[idx])
        if cumsum >= F(top_p):
            length = i + 1
            break
    if top_k > 0:
        length = min(length, top_k)
    inv_t = F(F(1.0) / temperature)
    top = [F(np.power(probs[idx], inv_t)) for idx in order[:length]]
    total = F(0)
    for v in top:  # std::accumulate with a float initial value
        total = F(total + v)
    r = F(1.0 * (gen() - gen.min) / (gen.max - gen.min) * float(total))
    cumsum = F(0)
    for i, v in enumerate(top):
        cumsum = F(cumsum + v)
        if cumsum >= r:
            return order[i]
    raise RuntimeError("cumulative scan ended below the draw")


class Penalties:
    """The repetition penalties of the reference's generation loop (chat.cpp:22-24, 40, 57-62, 77), in the
    loop's own arithmetic: before every draw, each token drawn so far (in ascending id order, the order of
    the std::map) has `frequency * count + presence` subtracted from its fp32 logit, the product and the sum
    evaluated in fp32, and its count is then multiplied by `decay`; the drawn token's count goes up by one."""

    def __init__(self, presence=0.8, frequency=0.8, decay=0.996):
        self.presence, self.frequency, self.decay = F(presence), F(frequency), F(decay)
        self.count = {}

    def apply(self, logits):
        """Adjusts `logits` (fp32 array) in place and decays the counts (chat.cpp:57-62)."""
        for tok in sorted(self.count):
            c = self.count[tok]
            logits[tok] = F(logits[tok] - F(F(self.frequency * c) + self.presence))
            self.count[tok] = F(c * self.decay)
        return logits

    def drawn(self, tok):
        """chat.cpp:77: `occurences[output_id]++`."""
        self.count[tok] = F(self.count.get(tok, F(0)) + F(1))
