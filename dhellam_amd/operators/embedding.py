"""Vocab-parallel word embedding: dhellam/operators/embedding.py:16-49.

Same calling convention as the reference (a dict in, a dict out, ``bwd(context, dout)`` with
``context = [inputs, outputs]`` as built by ``template_fwd``).  The reference's backward goes
through autograd and leaves the gradient in ``vocab.grad``; here it is accumulated by a
deterministic kernel into ``vocab.main_grad`` when the parameter has one (fp32 or the
parameter's type), else into ``vocab.grad``.
"""
from __future__ import annotations

from typing import Sequence

import torch

from .. import _lib
from ..common.parallel_state import get_tensor_model_parallel_rank, get_tensor_model_parallel_world_size


def vocab_range_from_per_partition_vocab_size(per_partition_vocab_size: int, rank, world_size: int) -> Sequence[int]:
    index_f = rank * per_partition_vocab_size
    return index_f, index_f + per_partition_vocab_size


def _vocab_start(vocab) -> int:
    # with one rank every id is inside the table, as in the reference's unmasked branch (embedding.py:30-31)
    return vocab_range_from_per_partition_vocab_size(vocab.shape[0], get_tensor_model_parallel_rank(),
                                                     get_tensor_model_parallel_world_size())[0]


def word_embedding_fwd(inputs):
    vocab, token_ids = inputs["vocab"], inputs["token_ids"]
    _lib.need_cuda(vocab, token_ids)
    assert vocab.dim() == 2 and vocab.is_contiguous() and token_ids.dtype == torch.int64
    ids = token_ids.contiguous()
    out = torch.empty(*ids.shape, vocab.shape[1], dtype=vocab.dtype, device=vocab.device)
    _lib.check(_lib.load().dh_embedding_fwd(vocab.data_ptr(), ids.data_ptr(), ids.numel(), vocab.shape[1],
                                            vocab.shape[0], _vocab_start(vocab), _lib.dt(vocab), out.data_ptr(),
                                            torch.cuda.current_stream().cuda_stream))
    return {"word_embeddings": out}


def word_embedding_bwd(context, dout):
    inputs = context[0]
    vocab, ids = inputs["vocab"], inputs["token_ids"].contiguous()
    _lib.need_cuda(vocab, dout)
    dout = dout.contiguous()
    assert dout.dtype == vocab.dtype and dout.numel() == ids.numel() * vocab.shape[1]
    grad = getattr(vocab, "main_grad", None)
    if grad is None:
        if vocab.grad is None:
            vocab.grad = torch.zeros_like(vocab)
        grad = vocab.grad
    assert grad.is_contiguous() and grad.shape == vocab.shape
    _lib.check(_lib.load().dh_embedding_bwd(dout.data_ptr(), ids.data_ptr(), ids.numel(), vocab.shape[1],
                                            vocab.shape[0], _vocab_start(vocab), _lib.dt(dout), grad.data_ptr(),
                                            _lib.dt(grad), torch.cuda.current_stream().cuda_stream))
    return None


def pos_embedding():
    pass
