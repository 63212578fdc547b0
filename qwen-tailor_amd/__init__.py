"""MI355X-native GatedDeltaNet + GQA-hd256 attention hot path (drop-in for the operators of wang90063/Qwen-tailor's
qwen35/gated_delta.py, gdn_nax.py, kernels.deltanet, batch.py, batch_spec.py and prefill.py on torch-ROCm tensors)."""
from . import _build, _lib  # noqa: F401
from . import model, gated_delta, gdn_nax, kernels, batch, batch_spec, prefill, attention, prefix_cache  # noqa: F401

__all__ = ["model", "gated_delta", "gdn_nax", "kernels", "batch", "batch_spec", "prefill", "attention"]
