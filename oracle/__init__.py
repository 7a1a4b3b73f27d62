"""CPU restatement of the reference's grouped-GEMM hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory: it exists so that tests, the smoke check and the benchmark's
``cpu_baseline`` leg have an independent checker for the HIP kernels.

Parity status of each restated function (what pins it):

* ``layout_ref``       pinned by the reference's seven known-answer tests
                       (tests/test_layout_backend.py:22-52) and closed forms.
* ``gemm_ref``         textbook per-group matmul; pinned by reduction to
                       ``torch.matmul`` / ``torch.bmm`` special cases.
* ``fp8_soft``         pinned exhaustively against the CPU ``torch`` cast for
                       every bf16 bit pattern and by the format's closed form.
* ``quant_ref``        128x128 transposing quantizer and the 1x128 / 128x128
                       cast recipes: pinned by brute-force per-element loops on
                       tiny inputs and by dequantisation invariants.
* block-scaled FP8 GEMM (``gemm_ref.fp8_block_scaled_reference``): the
  arithmetic lives in the un-vendored third-party ``deep_gemm`` package
  (no version pinned by the reference; call site gemm/deep_gemm_ops.py:99) and
  no reference test covers it -> **parity unpinned** by the reference; it is
  anchored on the closed form "fp32 matmul of the dequantised operands".
"""
