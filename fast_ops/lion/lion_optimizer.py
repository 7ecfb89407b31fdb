"""``fast_ops.lion.lion_optimizer`` - same names as the reference module of that path."""
from fast_ops_amd.lion.lion_optimizer import Lion, lion_update  # noqa: F401
