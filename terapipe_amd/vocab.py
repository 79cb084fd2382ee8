"""The two ends of the layer stack at tensor-parallel size 1: token embedding, LM head, vocabulary
cross-entropy.  Mirrors mpu.VocabParallelEmbedding (reference mpu/layers.py:85-141) and
mpu.vocab_parallel_cross_entropy (mpu/cross_entropy.py:25-110); every arithmetic step is a call into
libterapipe_hip.so through terapipe_amd.ops.
"""
import torch
import torch.nn as nn
from torch.nn import init

from . import ops
from ._lib import TP_EPI_STORE, TP_GEMM_NN, TP_GEMM_NT, TP_GEMM_TN


class _EmbeddingFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, ids, weight):
        flat = ids.reshape(-1).contiguous()
        out = ops.embedding_fwd(flat, weight)
        ctx.save_for_backward(flat)
        ctx.wshape, ctx.wdtype = weight.shape, weight.dtype
        return out.view(*ids.shape, weight.shape[1])

    @staticmethod
    def backward(ctx, dout):
        (flat,) = ctx.saved_tensors
        acc = torch.empty(ctx.wshape, dtype=torch.float32, device=dout.device)
        ops.zero_(acc)
        ops.embedding_bwd(flat, dout.reshape(flat.numel(), -1).contiguous(), acc)
        if ctx.wdtype == torch.float32:
            return None, acc
        dw = torch.empty(ctx.wshape, dtype=ctx.wdtype, device=dout.device)
        ops.accum_cast(dw, acc, False)
        return None, dw


class VocabParallelEmbedding(nn.Module):
    """mpu.VocabParallelEmbedding at tensor-parallel size 1 (the vocabulary range is the whole vocabulary,
    mpu/layers.py:108-113; the all-reduce of :139 is the identity)."""

    def __init__(self, num_embeddings, embedding_dim, init_method=init.xavier_normal_, device=None, dtype=None):
        super().__init__()
        self.num_embeddings, self.embedding_dim = num_embeddings, embedding_dim
        self.padding_idx, self.max_norm, self.norm_type = None, None, 2.0
        self.scale_grad_by_freq, self.sparse = False, False
        self.vocab_start_index, self.vocab_end_index = 0, num_embeddings
        self.num_embeddings_per_partition = num_embeddings
        self.weight = nn.Parameter(torch.empty(num_embeddings, embedding_dim, device=device, dtype=dtype))
        init_method(self.weight)

    def forward(self, input_):
        return _EmbeddingFunction.apply(input_, self.weight)


VOCAB_PAD = 64      # the 256-row GEMM tiles take whole 64-wide k-tiles: the data-gradient GEMM has k = vocabulary


def _pad_vocab(n):
    return (n + VOCAB_PAD - 1) // VOCAB_PAD * VOCAB_PAD


class _LMHeadFunction(torch.autograd.Function):
    """logits = h W^T with the vocabulary padded to a multiple of 64 columns for the GEMMs (the padding rows
    of the weight copy are zero; the padding columns of the logits are ignored by the loss)."""

    @staticmethod
    def forward(ctx, h2d, weight):
        V, E = weight.shape
        Vp = _pad_vocab(V)
        wp = weight
        if Vp != V:
            wp = torch.zeros(Vp, E, dtype=weight.dtype, device=weight.device)
            wp[:V].copy_(weight)
        h2d = h2d.contiguous()
        logits = torch.empty(h2d.shape[0], Vp, dtype=h2d.dtype, device=h2d.device)
        ops.gemm(TP_GEMM_NT, h2d, wp, h2d.shape[0], Vp, E, C=logits, epilogue=TP_EPI_STORE)
        ctx.save_for_backward(h2d, wp)
        ctx.V = V
        return logits

    @staticmethod
    def backward(ctx, dlogits):
        h2d, wp = ctx.saved_tensors
        M, E = h2d.shape
        Vp = wp.shape[0]
        dlogits = dlogits.contiguous()
        dh = torch.empty_like(h2d)
        ops.gemm(TP_GEMM_NN, dlogits, wp, M, E, Vp, C=dh)
        dwp = torch.empty_like(wp)
        ops.gemm(TP_GEMM_TN, dlogits, h2d, Vp, E, M, C=dwp)
        return dh, dwp[:ctx.V]


def lm_head_logits(h2d, weight):
    """[M, E] x [V, E]^T -> [M, V rounded up to a multiple of 64]; columns >= V are padding (see vocab_parallel_cross_entropy's
    `vocab_size`).  The usual GPT weight tying passes the embedding weight."""
    return _LMHeadFunction.apply(h2d, weight)


class _CrossEntropyFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, target, vocab_size):
        shape = target.shape
        l2 = logits.reshape(-1, logits.shape[-1])
        if not l2.is_contiguous():
            raise ValueError("vocab_parallel_cross_entropy overwrites its logits in place and needs them contiguous")
        loss = ops.cross_entropy_(l2, target.reshape(-1).contiguous(), vocab_size, 1.0)
        # l2 now holds softmax - onehot, as the reference keeps its softmax (:74).  The overwrite goes through
        # the raw pointer: the logits are the output of a GEMM whose backward does not read them.
        ctx.g2 = l2.detach()
        ctx.lshape = logits.shape
        return loss.view(shape)

    @staticmethod
    def backward(ctx, grad_output):
        g2 = ctx.g2
        ops.scale_rows_(g2, grad_output.reshape(-1).to(torch.float32).contiguous())
        return g2.view(ctx.lshape), None, None


def vocab_parallel_cross_entropy(vocab_parallel_logits, target, vocab_size=None):
    """Per-token loss log(sum exp logits) - logits[target] (mpu/cross_entropy.py:109-110).  Like the reference
    it overwrites the logits (there with the softmax, here directly with softmax - onehot).  vocab_size:
    number of valid leading columns when the logits come from lm_head_logits with a padded vocabulary."""
    V = vocab_parallel_logits.shape[-1] if vocab_size is None else vocab_size
    return _CrossEntropyFunction.apply(vocab_parallel_logits, target, V)
