"""palimpsa_amd: the Palimpsa attention operator as hand-written HIP kernels for
AMD MI355X (gfx950), behind the reference's own Python entry points.

    from palimpsa_amd.ops.palimpsa import chunk_palimpsa, fused_recurrent_palimpsa, palimpsa_ref
"""
__version__ = "0.1.0"
