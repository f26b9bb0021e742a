"""Sampling as the reference's Sampler does it (src/sampler.cpp): argmax with the
lowest index on ties, temperature sampling by a walk along the running sum,
and the probability of one token.  The arithmetic runs in HIP kernels over the
float32 logits on the device.  Randomness is explicit: the uniform number of a
draw is a function of (seed, request id, step) alone, so a request's tokens do
not depend on what else is in its batch (the reference seeds the C library's
global generator with the wall clock, src/main.cpp:66, src/sampler.cpp:6-9)."""
import torch

from ..ops import kernels

_MASK = (1 << 64) - 1


def _mix(x):
    x &= _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform(seed, request_id, step):
    """A number in [0, 1) with 24 random bits for draw `step` of request `request_id`."""
    h = _mix(_mix(_mix(seed * 0x9E3779B97F4A7C15 + 1) + request_id * 0xD1B54A32D192ED03 + 2) + step)
    return (h >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, seed=0):
        self.seed = int(seed)

    def sample(self, logits, temperature, request_ids, steps):
        """One token for each row of logits [R, vocab] (device, float32).
        temperature 0 is argmax.  Returns a list of ints."""
        R = logits.shape[0]
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
        if temperature == 0.0:
            kernels.argmax(logits, out)
        else:
            u = torch.tensor([uniform(self.seed, r, s) for r, s in zip(request_ids, steps)], dtype=torch.float32)
            kernels.sample(logits, u.to(logits.device), float(temperature), out)
        return out.tolist()

    def argmax(self, logits):
        out = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device)
        kernels.argmax(logits, out)
        return out.tolist()

    def prob(self, logits, index):
        """softmax(logits[r])[index[r]] at temperature 1 (src/sampler.cpp:11-25)."""
        idx = torch.tensor(list(index), dtype=torch.int32, device=logits.device)
        out = torch.empty(logits.shape[0], dtype=torch.float32, device=logits.device)
        kernels.token_prob(logits, idx, out)
        return out.tolist()
