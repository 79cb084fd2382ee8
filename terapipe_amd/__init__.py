"""MI355X-native implementation of TeraPipe's sliced GPT-layer hot path.

The public surface mirrors the reference's modules for this path:
``terapipe_amd.transformer_models`` (layer, attention with K/V cache, slicers) and
``terapipe_amd.terapipe`` (TransformerLayers, TeraPipe).  All arithmetic runs in the HIP kernels of
``libterapipe_hip.so`` (C ABI in include/terapipe_hip.h); there is no CPU or PyTorch-op fallback.
"""
from . import _lib  # noqa: F401
from .terapipe import TeraPipe, TransformerLayers, loss_func, uniform_slice  # noqa: F401
from .transformer_models import (MODEL_CONFIGS, BATCH_CONFIGS, NEG_INF, ColumnParallelLinear,  # noqa: F401
                                 ModelParallelMultiheadLMAttentionWithCache, ModelParallelTransformerLayer,
                                 MultiheadLMAttentionWithCache, RowParallelLinear, SingleDeviceTransformer,
                                 TransformerConfig, TransformerLayer, grid_slice_batch_and_sequence,
                                 uniform_slice_x)

__version__ = "0.1.0"
from .vocab import VocabParallelEmbedding, lm_head_logits, vocab_parallel_cross_entropy  # noqa: F401
from .optim import FusedAdam  # noqa: F401
