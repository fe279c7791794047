"""CPU oracle for the layer-wise quantization hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in ``lightcompress_amd`` imports this
package; only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` may call it, and there only as the checker / the timed CPU
baseline.  The product path has no CPU fallback: it raises when the HIP
library is missing.

Every function restates, on CPU tensors, the torch-op sequence (or the
published algorithm) of one reference function and cites it as
``file:line`` relative to ``llmc/compression/quantization/`` of
ModelTC/LightCompress.

Pinning status
--------------
* integer quantizer (``quant_ref.int_*``): pinned by closed forms, an
  independent numpy bit-level bf16 model, brute force in exact rational
  arithmetic and invariants (tests/test_oracle_quant.py).
* minifloat rounding (``quant_ref.float_quantize_nearest``): the grid is
  pinned against torch's own float8 casts on non-tie inputs and against
  exact rational arithmetic; the TIE RULE, subnormal handling and saturation
  belong to the third-party QPyTorch (``qtorch``, version unpinned by the
  reference's requirements/runtime.txt), whose source is not available here:
  **parity unpinned** for those three choices; they are parameters.
* what torch computes differently on its two platforms (0-dim tensor
  operands next to 16-bit tensors, the math library behind log2 / pow, the
  binning of histc, the mean of a reduction): the reference runs on the GPU,
  so the restatements follow torch's GPU kernels (``quant_ref.as_operand``,
  ``histc_device``, ``mean_rows``) and
  the ``-m gpu`` tests compare them, and the library, with the reference's
  expressions evaluated by torch on GPU tensors
  (tests/test_torch_gpu_semantics_gpu.py, test_quant_gpu.py).
* pack / gemm_pack: pinned by unpack round trips and brute force.
* GPTQ Hessian / Cholesky chain / column loop: pinned by fp64 closed forms
  and the loss identity  sum(Losses) == 1/2 tr((W0-Q) H (W0-Q)^T).
* AWQ: pinned by alpha=0 -> plain RTN, max*min==1 normalisation, brute force.
"""
