from fast_ops_amd.lion import Lion, lion_update  # noqa: F401
