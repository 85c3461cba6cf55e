"""Host-side mirror of ``mindspeed.ops`` for the MoE expert path."""
from .npu_moe_token_permute import npu_moe_token_permute, moe_token_permute_with_aux  # noqa: F401
from .npu_moe_token_unpermute import npu_moe_token_unpermute  # noqa: F401
from .gmm import npu_gmm, npu_gmm_v2, GMMFunction  # noqa: F401
from .npu_groupmatmul_add import npu_groupmatmul_add_fp32  # noqa: F401
from .swiglu import fused_swiglu, swiglu_with_probs  # noqa: F401
from .sort_chunks import sort_chunks_by_idxs  # noqa: F401
from .moe_permute_mask_map import MoePermuteMaskMap, MoeUnpermuteMaskMap  # noqa: F401
from .grouped_matmul import _GroupedMatmul, fused_grouped_matmul  # noqa: F401
from .te_grouped_linear import MindSpeedTEGroupedLinearGMM, MindSpeedTEGroupedLinear  # noqa: F401
from .gmm_swiglu import gmm_swiglu, GmmSwigluFunction, grouped_mlp, GroupedMLPFunction  # noqa: F401
