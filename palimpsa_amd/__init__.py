"""palimpsa_amd: the Palimpsa attention operator as hand-written HIP kernels for
AMD MI355X (gfx950), behind the reference's own Python entry points.

    from palimpsa_amd.ops.palimpsa import chunk_palimpsa, fused_recurrent_palimpsa, palimpsa_ref, DecodeStep
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla, fused_recurrent_simple_gla   # precision state off
    from palimpsa_amd.ops.layer_glue import palimpsa_inputs, palimpsa_output_norm         # the layer's element-wise work

Everything runs through libpalimpsa_hip.so (C ABI in include/palimpsa_hip.h, built by
``python -m palimpsa_amd.build``); there is no CPU or eager fallback.
"""
__version__ = "0.1.0"
