"""vectorlink_gpu on MI355X: the reference's Python surface over a hand-written HIP library."""
from .ann import ANN  # noqa: F401
from .queue import Queue  # noqa: F401
