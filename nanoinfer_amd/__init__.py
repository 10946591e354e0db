"""nanoinfer_amd: a small inference engine for one MI355X (gfx950).

From a model folder (``config.json`` + ``model.safetensors``) to next-token logits and generated
tokens: typed configuration and registries, weights by tensor name, parts assembled into a
model, a paged cache, one step function for mixed batches, a scheduler, samplers, and
hand-written HIP kernels under ``csrc/``.
"""
from . import registry
from .parts import standard as _standard_parts   # registers the parts
from .parts import hybrid as _hybrid_parts       # registers the parallel block, the mixers with a memory, routed experts
from .parts import stateful as _stateful_parts   # registers mixers with a state of fixed size, the windowed attention, the pair-hash embedding
from .parts import gated as _gated_parts         # registers the sandwich block, attention over keys or a latent, the gated matrix memory, the depth average
from .parts import postnorm as _postnorm_parts   # registers the postnorm block, attention with a sink, the capped feed-forward
from .architectures import llama as _llama       # registers LlamaForCausalLM
from .architectures import zekalorn as _zekalorn  # registers Zekalorn
from .architectures import fusavik as _fusavik    # registers Fusavik
from .architectures import ruludra as _ruludra    # registers Ruludra
from .architectures import vimilix as _vimilix    # registers Vimilix

__version__ = "0.1.0"
