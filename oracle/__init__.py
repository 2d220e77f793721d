"""CPU oracle for the attention hot path -- TEST INFRASTRUCTURE ONLY.

Everything under ``oracle/`` is a CPU restatement of the algorithms the reference
(Ascend/MindIE-SD) runs on this path.  It exists so the HIP kernels can be checked
against it.  Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` may import it; the product package never does, and the product
raises when its HIP library is missing instead of falling back to anything here.

Parity status of each function (what pins it, beyond re-typing its formula):

* ``attention.attention_math``          pinned: fp64 brute force on tiny inputs,
  ``torch.nn.functional.scaled_dot_product_attention`` in fp32, masked special cases.
* ``attention.block_sparse_attention``  pinned: all-ones mask == dense, empty row == 0,
  per-row dense attention over the gathered keys (brute force).
* ``rainfusion.window_order`` / ``rearrange`` / ``inv_rearrange``  pinned: the reference's
  einops pattern strings evaluated by einops on token ids, round trips on the reference's
  four grids, cross-check of two independent inverses.
* ``rainfusion.avgpool``                pinned: reference known answers (63.5 / 191.5),
  closed-form means, torch ``mean`` agreement.
* ``rainfusion.get_mask_index``         pinned: reference known answers.
* ``rainfusion.get_blockwise_mask``     pinned: torch ``einsum``/``softmax``/``topk`` composite
  in the same dtype (agreement up to floating-point summation-order ties, see its docstring),
  first-frame / text invariants, keep-count lower bound.
* ``quant.e4m3_round``                  pinned: all 256 codes + torch ``float8_e4m3fn`` casts.
* ``quant.dynamic_block_quant`` / ``mx_quant`` / ``fp8_attention`` / ``mxfp8_gemm_swiglu``
  PARITY UNPINNED against the reference: the reference delegates these to closed vendor ops
  (torch_npu) and mocks them in its own tests; they follow the published formats
  (OCP FP8 e4m3fn, OCP MX v1.0) and are pinned only against those definitions.
"""
