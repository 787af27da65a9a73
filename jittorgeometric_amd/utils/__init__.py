from .get_laplacian import get_laplacian  # noqa: F401
from .loop import add_remaining_self_loops, add_self_loops, remove_self_loops  # noqa: F401
from .num_nodes import maybe_num_nodes  # noqa: F401
