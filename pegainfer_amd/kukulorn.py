"""Python driver of the Kukulorn host runtime (libpegainfer_qwen3.so, include/pegainfer_kukulorn.h).

Kukulorn lists its layers one by one in config.json and walks a span of them several times on the same weights ("loop"), every
walk with a cache and state of its own; before every walk the stream is mixed with the embedding rows again.  A layer has one RMS
norm whose output the mixer and the feed-forward both read.  Mixers: "attention" (a short convolution over time on q, k and v,
rotation of the halves with long-context frequency scaling, unit-norm q and k, tanh-capped scores, a sigmoid gate per value) and
"parallel" (attention over a sliding window that keeps the first tokens, with a learned bias by distance, beside a selective
state-space layer; their normed outputs are averaged).  Feed-forward: relu(gate) * up.  Logits over the embedding table, capped.
A request holds cache pages AND a region of recurrent state; both are handed out again when it is dropped.
"""
from .step_engine import DTYPES, StepEngine  # noqa: F401


class KukulornEngine(StepEngine):
    architecture = "Kukulorn"
    prefix = "pegainfer_kukulorn_"

    def state_floats(self):
        """fp32 values of recurrent state one request holds"""
        return int(self._fn("state_floats")(self.h))
