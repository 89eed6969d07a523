"""Python driver of the Duguzen host runtime (libpegainfer_qwen3.so, include/pegainfer_duguzen.h).

Duguzen lists its layers one by one in config.json: latent-attention mixers (a compressed key/value latent plus one shared
rotated key part per token are all that is cached), Dynamic-Tanh norms around every sublayer over an fp32 residual stream,
dense squared-ReLU or sigmoid-routed SwiGLU feed-forwards, and layers that borrow another layer's weights.  The engine has
ONE step: prompts, portions of prompts and single decoded tokens of several requests run as one batch.  No CPU fallback.
"""
from .step_engine import DTYPES, StepEngine  # noqa: F401


class DuguzenEngine(StepEngine):
    architecture = "Duguzen"
    prefix = "pegainfer_duguzen_"
