from .interface import run_short_hyena  # noqa: F401
