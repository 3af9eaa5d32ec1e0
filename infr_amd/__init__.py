"""infr_amd — MI355X (gfx950) backend for infr's quantized-matmul path.

``infr_amd.backend`` mirrors infr-core's Backend seam over the C ABI declared in
``include/infr_hip.h``; ``infr_amd.build`` compiles the HIP sources into ``libinfr_hip.so``.
"""
from .backend import (  # noqa: F401
    Activation, Add, Bindings, Buffer, BufferUsage, DType, EmbedGather, GatedAct, GatedActFused, Graph, HipBackend,
    InfrError, Linear, MoeFfn, Plan, RmsNorm, RmsNormAdd, Status, TensorDesc, TensorId, block_layout,
    load_library, synth_normal_f32, synth_weight,
)
