"""MI355X-native kernel fusion for GPT-2 / GPT-Neo / GPT-J blocks: the fused
operator API of tunib-ai/oslo (``FusedScaleMaskSoftmax``, ``FusedBiasActivation``,
``FusedBiasDropout``, ``FusedBiasDropoutResidual``, ``model.fuse()``) on
hand-written gfx950 kernels behind a C ABI (``include/oslo_amd.h``)."""

from .fused_kernels_utils import (  # noqa: F401
    FusedBiasActivation,
    FusedBiasDropout,
    FusedBiasDropoutResidual,
    FusedBiasGeLU,
    FusedDecodeAttention,
    FusedPrefillAttention,
    FusedKernelMixin,
    FusedLinearBiasActivation,
    FusedLinearRows,
    FusedMergeHeads,
    FusedNoRepeatNGramLogitsProcessor,
    FusedRotaryPositionEmbedding,
    FusedScaleMaskSoftmax,
    FusedSplitHeads,
    FusedScaleMaskSoftmaxDropout,
    FusedScaleMaskWindowSoftmax,
    ScaledMaskedSoftmaxFunction,
    ScaledUpperTriangMaskedSoftmaxFunction,
    get_custom_kernels,
)
from .generation_utils import DynamicDecoder, GenerationMixin, StaticDecoder  # noqa: F401
from .graphs import GraphedForward  # noqa: F401
from .modeling_gpt2 import GPT2Config, GPT2LMHeadModel  # noqa: F401
from .modeling_gpt_neo import GPTNeoConfig, GPTNeoForCausalLM  # noqa: F401
from .modeling_gptj import GPTJConfig, GPTJForCausalLM  # noqa: F401
from .modeling_utils import DecodeState, StaticKV  # noqa: F401

__version__ = "0.1.0"
