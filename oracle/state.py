"""The transactional KV state crit's attention-state technique defines on the host, restated. Test infrastructure only:
nothing that ships may import this.

Follows inference/attention-state/code/implementation.py:5-50 (KVState): ordered committed and pending rows; stage()
appends to pending within capacity, commit(n) keeps the first n pending rows and drops the rest, rollback() drops them
all, attend() is a stable softmax over the committed rows (with include_pending: over all rows). Pinned
(tests/test_oracle.py) by the reference's known answers (README.md:224-238, tests/test_techniques.py:471-494: (6.0,) with
both staged rows, (2.0,) once one is committed, the errors) and by float64 attention over the same rows. On the device
the same transaction is a sequence's valid length: staged rows are written past it, a commit moves it, a rollback leaves
it (tests/test_gpu_pool.py drives both side by side).
"""
import math


class KVState:
    def __init__(self, capacity, key_width, value_width):
        for x in (capacity, key_width, value_width):
            if type(x) is not int or x <= 0:
                raise ValueError("positive integer state geometry required")
        self.capacity, self.key_width, self.value_width = capacity, key_width, value_width
        self.committed, self.pending = [], []

    def stage(self, key, value):
        key, value = tuple(key), tuple(value)
        if (len(key), len(value)) != (self.key_width, self.value_width):
            raise ValueError("KV geometry differs")
        if not all(math.isfinite(x) for x in key + value):
            raise ValueError("finite KV values required")
        if len(self.committed) + len(self.pending) >= self.capacity:
            raise ValueError("KV capacity exhausted")
        self.pending.append((key, value))

    def commit(self, count=None):
        if count is None:
            count = len(self.pending)
        if type(count) is not int or count < 0 or count > len(self.pending):
            raise ValueError("commit exceeds staged state")
        self.committed += self.pending[:count]
        self.pending = []

    def rollback(self):
        self.pending = []

    def attend(self, query, *, include_pending=False, scale=None):
        query = tuple(query)
        if len(query) != self.key_width or not all(math.isfinite(x) for x in query):
            raise ValueError("query geometry/domain differs")
        if scale is None:
            scale = 1 / math.sqrt(self.key_width)
        if not math.isfinite(scale) or scale <= 0:
            raise ValueError("positive finite attention scale required")
        rows = self.committed + (self.pending if include_pending else [])
        if not rows:
            raise ValueError("attention requires an admitted causal prefix")
        logits = [scale * sum(q * k for q, k in zip(query, key)) for key, _ in rows]
        top = max(logits)
        weights = [math.exp(x - top) for x in logits]
        total = sum(weights)
        return tuple(sum(w * value[c] for w, (_, value) in zip(weights, rows)) / total for c in range(self.value_width))
