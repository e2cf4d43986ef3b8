"""CPU oracle for the DHeLlam per-rank operator hot path.

TEST INFRASTRUCTURE ONLY.  These are plain eager restatements (PyTorch on the
CPU in fp64/fp32 for floating point, numpy for index work) of what each
operator on the path computes.  Only ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py`` may import this package, and only
as the checker or as the timed CPU baseline.  Nothing under ``dhellam_amd/``
imports it, and the product has no CPU path.

How each function is pinned (the reference ships no tests, golden vectors or
fixtures, and its arithmetic for most of this path lives in packages that are
not vendored: transformer-engine 1.4.0, flash-attn >= 2.0.6, Megatron-core
0.5.0):

* ``ops.swiglu_fwd / swiglu_bwd``     restated from dhellam/operators/swiglu.py:13-26;
  pinned by ``torch.nn.functional.silu`` and fp64 autograd, plus y1 = 0 special case.
* ``ops.norm_fwd / norm_bwd``         textbook RMSNorm / LayerNorm (the reference calls
  TE's kernel, dhellam/operators/layernorm.py:37,82); pinned by
  ``torch.nn.functional.rms_norm`` / ``layer_norm`` in fp64 and fp64 autograd.
* ``ops.rope``                        rotate-half closed form (absent from the reference);
  pinned by complex multiplication, norm preservation, R(p)R(q) = R(p+q), inverse.
* ``ops.bda_fwd / bda_bwd``           dhellam/operators/bda.py:3-12 with the dropout mask
  identically one.
* ``attention.attn_fwd / attn_bwd``   dense softmax attention; pinned by
  ``torch.logsumexp``, ``F.scaled_dot_product_attention`` and fp64 autograd.
* ``attention.ring_*`` / ``merge``    dhellam/operators/ring_attn.py:26-40,90-201,204-411;
  pinned by equality with ONE dense causal attention over the zig-zag token order.
* ``moe.*``                           numpy index arithmetic; pinned by brute force,
  ``numpy.argsort(kind="stable")``, bijection and round-trip invariants.
* ``layer.*``                         the decoder layer of configs 0 and 2 with autograd; pinned by an
  independently written forward from library routines (``F.rms_norm``, ``F.linear``,
  ``F.scaled_dot_product_attention``, ``F.silu``) with fp64 autograd at 1e-12, and the
  sequence-parallel gather / scatter stand-ins by explicit slicing.
* ``head.*``                          dhellam/operators/loss.py:15-164 and embedding.py:16-49, restated
  line by line; pinned by ``F.cross_entropy`` / ``F.embedding`` and their autograd, one rank and four.

Every function above is pinned by the checks named with it (``tests/test_oracle_pins.py``,
``tests/test_golden.py``).  None of them could be held against numbers produced by the
reference itself: it cannot run without CUDA, TransformerEngine, flash-attn and Megatron,
and it holds no recorded outputs.
"""
