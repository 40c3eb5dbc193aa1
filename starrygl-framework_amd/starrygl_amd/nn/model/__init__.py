from .time_encoder import TimeEncoder  # noqa: F401
