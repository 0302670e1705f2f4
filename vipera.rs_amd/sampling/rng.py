"""The seeded generator of the sampler: xorshift64* seeded through SplitMix64.

Same generator as the reference's (crates/vipera-sampler/src/rng.rs:13-57), so a seed names the
same stream of uniforms.  One generator belongs to one request; its state does not depend on what
else is in a batch.

While a request runs, the state of its generator lives on the device, in the request's state slot, and the
sampling kernel advances it.  This class is the same generator on the host: it turns a seed into the state a
slot starts with, winds a state forward by the draws a request has already made when it comes back into a
slot after a preemption, and serves the tests as an oracle.
"""
_MASK = (1 << 64) - 1


def _splitmix64(state: int) -> int:
    state = (state + 0x9E3779B97F4A7C15) & _MASK
    z = state
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


class Rng:
    __slots__ = ("state",)

    def __init__(self, seed: int = 0):
        self.state = _splitmix64((int(seed) ^ 0x9E3779B97F4A7C15) & _MASK)

    def next_u64(self) -> int:
        x = self.state
        x ^= x >> 12
        x ^= (x << 25) & _MASK
        x ^= x >> 27
        self.state = x
        return (x * 0x2545F4914F6CDD1D) & _MASK

    def skip(self, draws: int) -> "Rng":
        """Advance by ``draws`` outputs."""
        for _ in range(draws):
            self.next_u64()
        return self

    def next_f64(self) -> float:
        """Uniform in [0, 1) with 53 bits."""
        return (self.next_u64() >> 11) / 9007199254740992.0
