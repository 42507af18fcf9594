from .task import Task  # noqa: F401
