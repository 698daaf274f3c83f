"""Python driver of the Ramalix host runtime (libpegainfer_qwen3.so, include/pegainfer_ramalix.h).

Ramalix lists its layers one by one in config.json and walks a span of them several times on the same weights ("loop"), every
walk with a cache and state of its own.  Sublayers are pre-norm with a one-number RMS gain and a constant residual factor; what
a sublayer reads first gets a short causal convolution over time added to it.  Mixers: "attention" (two softmax maps per head
combined as a difference, normed per head), "attention_2" (pair rotation, keys inside the query's own block of positions, a
sink logit in the denominator) and "channel_delta" (gated delta rule with a decay per head and key channel).  Feed-forward:
SwiGLU experts behind a softmax router restricted to its best groups, plus a gated shared expert.
A request holds cache pages AND a region of recurrent state; both are handed out again when it is dropped.
"""
from .step_engine import DTYPES, StepEngine  # noqa: F401


class RamalixEngine(StepEngine):
    architecture = "Ramalix"
    prefix = "pegainfer_ramalix_"

    def state_floats(self):
        """fp32 values of recurrent state one request holds"""
        return int(self._fn("state_floats")(self.h))
