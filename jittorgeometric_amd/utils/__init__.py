from .loop import add_remaining_self_loops  # noqa: F401
from .num_nodes import maybe_num_nodes  # noqa: F401
