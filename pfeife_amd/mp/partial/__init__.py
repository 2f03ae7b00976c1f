from .module import PartialModule, PartialRunner, partial_compiler  # noqa: F401
