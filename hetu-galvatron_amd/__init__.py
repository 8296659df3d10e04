"""MI355X (gfx950) implementation of Hetu-Galvatron's MoE expert-layer hot path.

Python modules mirror the reference's (galvatron/core/runtime/moe/*, models/moe_modules.py); all
compute goes through libgalvatron_moe.so (hand-written HIP, C ABI in include/galvatron_moe.h).
"""
from . import _C, ops, configs  # noqa: F401
from .config import MoEConfig  # noqa: F401
from . import moe_utils, fused_kernels, grouped_gemm, router, mlp, token_dispatcher, moe_modules  # noqa: F401
from . import checkpoint, norm  # noqa: F401
from .moe_utils import permute, unpermute, sort_chunks_by_idxs, topk_softmax_with_capacity  # noqa: F401
from .fused_kernels import moe_permute, moe_unpermute, moe_sort_chunks_by_index  # noqa: F401
from .router import TopKRouter  # noqa: F401
from .mlp import GroupedMLP, SequentialMLP, SharedExpertMLP, Fp8GroupedMLP  # noqa: F401
from .token_dispatcher import MoEAllGatherTokenDispatcher, MoEAlltoAllTokenDispatcher  # noqa: F401
from .moe_modules import GalvatronMoERouter, GalvatronMoEMLP  # noqa: F401
from .norm import RMSNorm, GalvatronNorm, PreRouterNorm, rms_norm  # noqa: F401

__version__ = "0.1.0"
