"""PipeOption: the user-facing configuration object.

Same constructor keywords, attribute names, argparse flags and `from_args`
behaviour as the reference (pfeife/option.py:52-279), so existing training
scripts keep working.  Fields that only steer subsystems this executor does not
have (device benchmark files, reducer backend, FSDP, the auto-partitioner) are
accepted and stored but not acted on.

One extension: an entry of `split_points` may be a string.  It then names the
module path (as recorded by TorchDynamo, e.g. "blocks.12") whose first graph
node starts a new stage; integers index the compute nodes of the captured graph
in topological order (placeholders and the output node are not counted).
"""
import logging

import torch
import torch.optim as optim

from .utils import set_logger_level

default_optimizer = dict(type="adam", lr=1e-5)

_OPTIMIZERS = {
    "adam": optim.Adam,
    "adamw": optim.AdamW,
    "adagrad": optim.Adagrad,
    "adamax": optim.Adamax,
    "asgd": optim.ASGD,
    "rmsprop": optim.RMSprop,
    "rprop": optim.Rprop,
    "sgd": optim.SGD,
}


def get_optimizer_cls(optimizer_type):
    cls = _OPTIMIZERS.get(optimizer_type.lower())
    if cls is None:
        print("Unknown optimizer type: %s. Use SGD instead." % optimizer_type)
        return optim.SGD
    return cls


_PRECISIONS = {"fp16": torch.float16, "bf16": torch.bfloat16}
_VERBOSITY = {"error": logging.ERROR, "info": logging.INFO, "debug": logging.DEBUG}


class PipeOption:
    """
    compiler            dynamo backend for per-stage compilation (ignored: stages run on the HIP executor)
    optimizer           dict(type=..., **kwargs of the torch optimizer)
    device_cnt          number of pipeline ranks the schedule is drawn for (all run on one GPU here)
    batch_size          size of one micro-batch
    batch_cnt           number of micro-batches per step (default device_cnt)
    loop_cnt            stages per rank of a looped schedule
    loop_batch          micro-batches per loop of a looped schedule (default device_cnt)
    prefetch_fwd        extra forwards issued before the first backward (default 0)
    split_points        stage boundaries (see module docstring)
    mixed_precision     None | "fp16" | "bf16"
    verbosity           'error' | 'warning' | 'info' | 'debug'
    """

    def __init__(self, **kwargs):
        get = kwargs.get
        self.compiler = get("compiler", None)
        self.reducer_backend = get("reducer_backend", "nccl")
        self.cpu_test = get("cpu_test", False)

        self.device_cnt = get("device_cnt", 2)
        self.batch_size = get("batch_size", 4)
        self.batch_cnt = get("batch_cnt", self.device_cnt)

        self.loop_cnt = get("loop_cnt", None)
        self.loop_batch = get("loop_batch", None)
        self.prefetch_fwd = get("prefetch_fwd", None)
        self.split_points = get("split_points", None)
        self.bench_seed = get("bench_seed", 0)

        self.verbosity = get("verbosity", "info")
        self.print_graph = get("print_graph", False)
        self.device_map = get("device_map", ["cuda:%d" % i for i in range(self.device_cnt)])
        self.device_bench = get("device_bench", None)
        self.graph_bench = get("graph_bench", None)
        self.scheduler = get("scheduler", "single_comm")
        self.partitioner = get("partitioner", "beam_single")
        self.linearizer = get("linearizer", "none")
        self.use_fsdp = get("use_fsdp", False)
        self.mixed_precision = _PRECISIONS.get(get("mixed_precision", None), get("mixed_precision", None))

        # Loss scale, applied ONCE, to the gradients entering the last stage, and removed again
        # before the optimizer step (the reference's GradScaler scales at every stage, so its
        # stage i of L sees S^(L-i)).  "dynamic": torch.amp.GradScaler's rule (worker.py:133-145)
        # kept on the device: overflowing steps are skipped and halve the scale, `growth_interval`
        # clean steps double it.  A number: that static scale.  Default: dynamic for every mixed
        # precision, fp16 and bf16 alike, as the reference builds its GradScaler
        # (`enabled=mixed_precision is not None`, worker.py:135): a bf16 step whose gradients are
        # not finite is skipped too.  1.0 without mixed precision.
        ls = get("loss_scale", None)
        if ls is None:
            ls = "dynamic" if self.mixed_precision in (torch.float16, torch.bfloat16) else 1.0
        self.loss_scale = "dynamic" if isinstance(ls, str) and ls.lower() == "dynamic" else float(ls)
        self.init_scale = float(get("init_scale", 65536.0))
        self.growth_factor = float(get("growth_factor", 2.0))
        self.backoff_factor = float(get("backoff_factor", 0.5))
        self.growth_interval = int(get("growth_interval", 2000))

        self.no_side_effect = get("no_side_effect", False)
        self.no_io_cache = get("no_io_cache", False)
        self.single_comm_thread = get("single_comm_thread", False)
        self.no_bench_optimizer = get("no_bench_optimizer", False)

        self.verbosity = _VERBOSITY.get(self.verbosity, logging.WARNING)

        optimizer = dict(get("optimizer", default_optimizer))
        self.optimizer_type = optimizer.pop("type")
        self.optimizer_kwargs = optimizer

    @staticmethod
    def from_args(args):
        if args.old_ver:
            args.no_side_effect = True
            args.no_io_cache = True
            args.single_comm_thread = True
        if args.cpu:
            args.single_comm_thread = True

        device_map = None
        if args.device_map:
            text = args.device_map.strip()
            if ":" in text:
                start, end = text.split(":")
                ids = range(int(start), int(end))
            else:
                ids = [int(t) for t in text.split(",")]
            device_map = ["cuda:%d" % i for i in ids]

        split_points = None
        if args.split_points:
            split_points = []
            for tok in args.split_points.strip().split(","):
                tok = tok.strip()
                split_points.append(int(tok) if tok.lstrip("-").isdigit() else tok)

        option_kwargs = dict(
            compiler=args.backend,
            reducer_backend=args.reducer_backend,
            device_cnt=args.device_cnt,
            loop_cnt=args.loop_cnt,
            loop_batch=args.loop_batch,
            prefetch_fwd=args.prefetch_fwd,
            split_points=split_points,
            batch_size=args.batch_size,
            batch_cnt=args.batch_cnt,
            use_fsdp=args.use_fsdp,
            mixed_precision=args.mixed_precision,
            optimizer={"type": args.optimizer_type, "lr": 1e-3},
            scheduler=args.scheduler,
            partitioner=args.partitioner,
            linearizer=args.linearizer,
            device_bench=args.device_bench,
            graph_bench=args.graph_bench,
            verbosity="debug" if args.verbose else "info",
            bench_seed=0,
            cpu_test=args.cpu,
            print_graph=args.print_graph,
            no_bench_optimizer=args.no_bench_optimizer,
            no_side_effect=args.no_side_effect,
            no_io_cache=args.no_io_cache,
            single_comm_thread=args.single_comm_thread,
        )
        if getattr(args, "loss_scale", None) is not None:
            option_kwargs["loss_scale"] = args.loss_scale
        if device_map is not None:
            option_kwargs["device_map"] = device_map

        option = PipeOption(**option_kwargs)
        option.set_logger()
        return option

    def set_logger(self):
        set_logger_level(self.verbosity)

    @staticmethod
    def add_arguments(parser):
        add = parser.add_argument
        add("--backend", help="backend for dynamo compiler")
        add("--reducer_backend", default="nccl", choices=["nccl", "gloo"], help="backend for gradient reducer")
        add("--verbose", action="store_true")
        add("--device_cnt", type=int, default=2, help="Size of pipeline parallelism")
        add("--batch_size", type=int, default=2)
        add("--batch_cnt", type=int, default=4)
        add("--optimizer_type", default="adam")
        add("--use_fsdp", action="store_true")
        add("--mixed_precision", choices=["fp16", "bf16"], default=None)
        add("--bench_seed", type=int, help="set seed for benchmarking. if 0, do not set seed.")
        add("--scheduler", choices=["single_comm", "beam", "dfs", "bfs", "pipeless"], default="single_comm")
        add("--partitioner", choices=["beam_single", "beam_2", "random_walk", "same_mem", "same_time"],
            default="beam_single")
        add("--linearizer", choices=["save_mem", "short_first", "long_first", "none"], default="none")
        add("--device_map", help="select usable devices. e.g. '0:3', '1,2,5,6'")
        add("--device_bench", help="path to device benchmark file. If there is no file, create one.")
        add("--graph_bench", help="path to ComputationGraph benchmark file. If there is no file, create one.")
        add("--cpu", action="store_true", help="run on cpu (test only)")
        add("--split_points", help="set split points for the pipe graph. e.g. '10,15,20' or 'blocks.12'")
        add("--loop_cnt", type=int,
            help="loop the forward pass by loop_cnt. If not set, find the best loop_cnt automatically.")
        add("--loop_batch", type=int, help="how many micro-batches in a single loop. If not set, find it automatically.")
        add("--prefetch_fwd", type=int,
            help="how many forward passese should be prefetched. If not set, find it automatically.")
        add("--no_bench_optimizer", action="store_true",
            help="run an optimizer when running computation graph benchmark")
        add("--no_side_effect", action="store_true", help="turn off dynamo side-effect")
        add("--no_io_cache", action="store_true",
            help="do not create io cache and send new tensor every time by tensor.to")
        add("--single_comm_thread", action="store_true", help="use single communication thread for all devices.")
        add("--old_ver", action="store_true", help="apply the above three actions.")
        add("--print_graph", action="store_true")
        add("--loss_scale", default=None,
            help="'dynamic' (GradScaler's rule, the default with --mixed_precision fp16) or a fixed number")
        return parser
