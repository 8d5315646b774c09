"""MI355X-native attention hot path for AR-TabPFN (shared-context decode,
teacher-forced log-density, context prefill) behind the reference's attention and
KV-cache interface.  The kernels are hand-written HIP for gfx950 reached through a
C ABI (``include/artab_attention.h``); this package is the host-side mirror of the
reference's Python callables."""

from .attention_kernels import (  # noqa: F401
    buffer_attention,
    context_attention,
    cross_attention,
    decode_attention,
    hip_available,
    hybrid_attention,
    hybrid_teacher_forcing_attention,
    merge_attention_outputs,
    prefill_attention,
    pytorch_buffer_attention,
    pytorch_context_attention,
    pytorch_teacher_forcing_buffer_attention,
    teacher_forcing_attention,
    teacher_forcing_buffer_attention,
    triton_available,
    triton_context_attention,
)

from .attention import (  # noqa: F401,E402
    DecodeMask,
    DenseMask,
    MultiheadAttention,
    TeacherForcingMask,
    clear_mask_cache,
    create_context_self_attention_mask,
    create_dense_mask,
    create_row_mask,
)
from .inference import ARTabPFNPredictor  # noqa: F401,E402
from .model import (  # noqa: F401,E402
    ARTabPFN,
    Embedder,
    MixtureGaussianHead,
    TwoStageTransformer,
    TwoStageTransformerLayer,
)

__version__ = "0.1.0"
