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


class Drawn:
    """The tokens of one draw: on the device at once (`tokens`, int32 [R]), on the host once the
    copy that follows the sampling kernel has landed (`tolist()` waits for it, and for nothing
    that was queued later)."""

    def __init__(self, tokens, host, landed, sampler, turn):
        self.tokens = tokens
        self._host = host
        self._landed = landed
        self._sampler, self._turn = sampler, turn
        self._list = None

    def tolist(self):
        if self._list is None:
            if self._sampler._turn - self._turn >= Sampler.HOST_BUFFERS:
                raise RuntimeError("the tokens of a draw are read after %d later draws have taken its host buffer"
                                   % Sampler.HOST_BUFFERS)
            self._landed.synchronize()
            self._list = self._host.tolist()
        return self._list


class Sampler:
    HOST_BUFFERS = 4          # draws whose host copies may be unread at the same time

    def __init__(self, seed=0):
        self.seed = int(seed)
        self._host = []           # pinned buffers and the events after the copies into them, used in turn
        self._turn = 0

    def _host_buffers(self, R):
        """The next pinned pair in turn: int32 for the tokens on their way back, float32 for the
        uniform numbers on their way out, and the event behind the draw that used them last."""
        if len(self._host) < self.HOST_BUFFERS:
            n = max(R, 64)
            self._host.append([torch.empty(n, dtype=torch.int32, pin_memory=True),
                               torch.empty(n, dtype=torch.float32, pin_memory=True), torch.cuda.Event()])
            return self._host[-1]
        entry = self._host[self._turn % self.HOST_BUFFERS]
        entry[2].synchronize()
        if entry[0].shape[0] < R:
            entry[0] = torch.empty(R, dtype=torch.int32, pin_memory=True)
            entry[1] = torch.empty(R, dtype=torch.float32, pin_memory=True)
        return entry

    def draw(self, logits, temperature, request_ids, steps):
        """One token for each row of logits [R, vocab] (device, float32); temperature 0 is argmax.
        Nothing waits for the device here: the tokens can feed the next step from where they lie
        while the host reads them a step later."""
        R = logits.shape[0]
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
        host, host_u, landed = self._host_buffers(R)
        if temperature == 0.0:
            kernels.argmax(logits, out)
        else:
            host_u[:R] = torch.tensor([uniform(self.seed, r, s) for r, s in zip(request_ids, steps)],
                                      dtype=torch.float32)
            u = torch.empty(R, dtype=torch.float32, device=logits.device)
            u.copy_(host_u[:R], non_blocking=True)          # from pinned memory: the host does not wait for the queue
            kernels.sample(logits, u, float(temperature), out)
        host[:R].copy_(out, non_blocking=True)
        landed.record()
        self._turn += 1
        return Drawn(out, host[:R], landed, self, self._turn)

    def sample(self, logits, temperature, request_ids, steps):
        """As draw, but returns the tokens as a list of ints."""
        return self.draw(logits, temperature, request_ids, steps).tolist()

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
