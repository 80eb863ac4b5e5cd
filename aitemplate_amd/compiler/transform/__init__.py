from .memory_planning import memory_planning  # noqa: F401
from .name_graph import name_graph  # noqa: F401
from .profile import profile  # noqa: F401
from .refine_graph import refine_graph  # noqa: F401
from .toposort import toposort  # noqa: F401
from .mark_param_tensor import mark_param_tensor  # noqa: F401
from .transform_utils import get_sorted_ops  # noqa: F401
from .fuse_mm_elementwise import check_leftover_elementwise, fuse_mm_elementwise  # noqa: F401
from .fuse_strided_views import fuse_strided_views  # noqa: F401
