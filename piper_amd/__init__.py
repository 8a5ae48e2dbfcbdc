"""piper_amd: the per-device compute of one Piper stage on AMD MI355X (gfx950).

Hot path only: the MoE expert region (router top-k, permute, grouped SwiGLU experts, combine;
forward and backward) and the ZeRO bucket path (flatten, gradient pack, fused AdamW, unflatten),
behind Piper's annotate / task / operator surface.  The kernels live in libpiper_amd.so
(C ABI: include/piper_amd.h); there is no CPU or PyTorch fallback.
"""
from .annotate import EP_TAG, PP_TAG, annotate, current_annotations, current_tag, reset_annotation_state
from .tasks import TaskType

__all__ = [
    "annotate", "current_annotations", "current_tag", "reset_annotation_state", "PP_TAG", "EP_TAG",
    "TaskType",
]
__version__ = "0.1.0"
