"""pfeife_amd: MI355X-native executor for Pfeife's pipeline-stage hot path.

Public names mirror the reference package (`pfeife/__init__.py:1`,
`pfeife/mp/__init__.py:1-8`)."""
from .option import PipeOption  # noqa: F401
