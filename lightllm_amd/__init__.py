"""MI355X-native (gfx950) block-FP8 W8A8 linear path behind LightLLM's operator interface.

The package holds only what that path needs:

* ``csrc/``           hand-written HIP kernels and the C ABI (``include/mi355_fp8.h``)
* ``_lib``            ctypes binding of ``lib/libmi355fp8.so``
* ``quantization/``   ``per_token_group_quant_fp8``, ``w8a8_block_fp8_matmul``, ``weight_quant`` and the
                      ``QuantizationMethod`` plug-in classes, with LightLLM's names and signatures
* ``fused_moe/``      ``moe_align_fused``, ``moe_align2``, ``grouped_matmul`` for ragged per-expert batches

There is no CPU or eager fallback: every operator raises if the HIP library cannot be loaded.
"""
__version__ = "0.1.0"
