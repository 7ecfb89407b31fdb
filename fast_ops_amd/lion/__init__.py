from .lion_optimizer import Lion, lion_update  # noqa: F401
