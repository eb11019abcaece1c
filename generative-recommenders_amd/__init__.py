"""MI355X-native HSTU jagged attention (forward): ``hstu_mha`` and ``delta_hstu_mha``, the jagged
concatenation / split that feeds the cached form (``concat_2D_jagged``, ``split_2D_jagged``, ``write_kv_tail``),
and the dense steps either side of the attention (``hstu_compute_uqvk``, ``hstu_compute_output``,
``hstu_preprocess_and_attention``).

Drop-in for ``generative_recommenders.ops.hstu_attention`` of the reference, backed by
hand-written gfx950 HIP kernels behind a C ABI (``csrc/``, ``include/hstu_hip.h``).
The directory name contains a hyphen, so load it with ``importlib`` under the module name
``generative_recommenders_amd`` (``__graft_entry__.load_package()`` does exactly that).
"""

from .common import HammerKernel  # noqa: F401
from .ops.hstu_attention import delta_hstu_mha, hstu_mha  # noqa: F401
from .ops.hstu_compute import hstu_compute_output, hstu_compute_uqvk, hstu_preprocess_and_attention  # noqa: F401
from .ops.jagged_tensors import concat_2D_jagged, split_2D_jagged, write_kv_tail  # noqa: F401
from .ops import native_op  # noqa: F401  (defines torch.ops.hstu.hstu_mha / hstu_mha_fwd on these kernels)

__all__ = [
    "HammerKernel", "hstu_mha", "delta_hstu_mha", "concat_2D_jagged", "split_2D_jagged", "write_kv_tail", "hstu_compute_uqvk",
    "hstu_compute_output", "hstu_preprocess_and_attention",
]
