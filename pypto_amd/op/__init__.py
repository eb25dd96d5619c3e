from .comparison import topk  # noqa: F401
