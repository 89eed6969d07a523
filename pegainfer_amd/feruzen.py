"""Python driver of the Feruzen host runtime (libpegainfer_qwen3.so, include/pegainfer_feruzen.h).

Feruzen lists its layers one by one in config.json.  Every layer adds a short causal convolution over time to the mixer's
input, norms the sublayers' OUTPUTS in groups before the residual sum (fp32 stream), and hands on a learned weighted sum over
the streams of all layers so far.  Mixers: "delta" (gated delta rule over a per-request matrix state, short convolutions on
q / k / v) and "parallel" (softmax attention with grouped key/value heads over the paged cache beside an exponentially gated
matrix memory).  Feed-forward: clamped gated-linear units, dense or routed by a softmax router with a shared expert.
A request holds cache pages AND a region of recurrent state; both are handed out again when it is dropped.
"""
from .step_engine import DTYPES, StepEngine  # noqa: F401


class FeruzenEngine(StepEngine):
    architecture = "Feruzen"
    prefix = "pegainfer_feruzen_"

    def state_floats(self):
        """fp32 values of recurrent state one request holds"""
        return int(self._fn("state_floats")(self.h))
