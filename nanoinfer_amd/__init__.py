"""nanoinfer_amd: a small inference engine for one MI355X (gfx950).

From a model folder (``config.json`` + ``model.safetensors``) to next-token logits and generated
tokens: typed configuration and registries, weights by tensor name, parts assembled into a
model, a paged cache, one step function for mixed batches, a scheduler, samplers, and
hand-written HIP kernels under ``csrc/``.
"""
from . import registry
from .parts import standard as _standard_parts   # registers the parts
from .architectures import llama as _llama       # registers LlamaForCausalLM

__version__ = "0.1.0"
