"""Import-path alias: scripts written for MerHS/pfeife (`from pfeife import PipeOption`,
`from pfeife.mp import initialize_pfeife, PartialRunner, partial_compiler`,
`from pfeife.loss import ...`, `from pfeife.batch import split_args_kwargs`) run unchanged on
the MI355X executor in `pfeife_amd`.  Module layout mirrored: pfeife/__init__.py:1,
pfeife/mp/__init__.py:1-8 of the reference."""
import importlib
import sys

import pfeife_amd
from pfeife_amd import PipeOption  # noqa: F401

for _name in ("option", "batch", "loss", "utils", "mp", "mp.net_states", "mp.partial", "mp.partial.module",
              "mp.worker", "schedule", "schedule.scheduler", "graph", "graph.partition_graph"):
    sys.modules["pfeife." + _name] = importlib.import_module("pfeife_amd." + _name)

mp = sys.modules["pfeife.mp"]
option = sys.modules["pfeife.option"]
batch = sys.modules["pfeife.batch"]
loss = sys.modules["pfeife.loss"]
