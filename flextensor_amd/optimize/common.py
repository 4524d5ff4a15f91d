"""Shared pieces of the tuning drivers: argument parser, evaluate, test.

Same roles and command-line flags as the reference's
flextensor/optimize/common.py (evaluate :17-60, test :63-82,
init_arg_parser :85-114). ``--check`` compares the tuned kernels with the
plain default-schedule kernels of the same task on the device, which is what
the reference's ``check_result`` does with the default llvm build, and runs
the static check of the kernels' assembly (isa_check).
"""
import os
import sys

from ..measure import WrongResult, get_measurer
from ..scheduler import schedule_with_config
from ..task import TASK_TABLE


def evaluate(name, s, bufs, target, dev_id, number=10, rpc_info=None, result_generator=None):
    """Mean ms of plan ``s`` over ``number`` launches; ``inf`` on failure."""
    if rpc_info is not None and getattr(rpc_info, "use_rpc", None):
        raise RuntimeError("remote measurement is not supported by the gfx950 backend")
    try:
        return get_measurer(s.task_key).evaluate(s, number=number)
    except Exception as e:  # noqa: BLE001
        print(e)
        return float("inf")


def test(task_key, configs, dev_id=None, rpc_info=None, check_result=False):
    """Replay ``configs`` and time them (every run passes the on-device
    correctness gate; ``check_result`` additionally prints the metric)."""
    task = TASK_TABLE[task_key]
    s, bufs = schedule_with_config(task_key, configs)
    dev_id = dev_id if dev_id is not None else task.dev_id
    time_cost = evaluate(task_key, s, bufs, task.target, dev_id, 100, rpc_info)
    if check_result:
        # against the default-schedule kernels on the device, then the static checks of the assembly
        try:
            print("Test correctness...", "passed!", "metric", s.verify(static=False))
        except WrongResult as e:
            print("Test correctness...", "failed!", e)
        from .. import isa_check
        if os.path.exists(isa_check.HIPCC):
            early = isa_check.check_plan(s)
            print("Test instruction stream...", "passed!" if not early else "failed! %s" % (early[:2],))
    print(task_key, "use", time_cost, "ms")
    print()
    return time_cost


test.__test__ = False


def init_arg_parser(parser):
    parser.add_argument("-f", "--from_", help="From which shape", type=int, default=0)
    parser.add_argument("-t", "--to", help="To which shape", type=int, default=-1)
    parser.add_argument("-l", "--log", help="Log file name", type=str, default="")
    parser.add_argument("--test", help="test file name", type=str, default="")
    parser.add_argument("--trials", help="number of trials for op", type=int, default=100)
    parser.add_argument("--target", help="target device type", type=str, default="rocm")
    parser.add_argument("--device", help="target device number", type=int, default=0)
    parser.add_argument("--timeout", help="timeout", type=int, default=4)
    parser.add_argument("--parallel", help="compile workers", type=int, default=1)
    parser.add_argument("--use_model", help="use performance model", action="store_true")
    parser.add_argument("--method", help="how to schedule", type=str, default="searching")
    parser.add_argument("--slevel", type=int, default=4)
    parser.add_argument("--rlevel", type=int, default=3)
    parser.add_argument("--force_inline", action="store_true")
    parser.add_argument("--host", type=str, default="0.0.0.0")
    parser.add_argument("--target_host", type=str, default="llvm")
    parser.add_argument("--device_key", type=str, default="")
    parser.add_argument("--use_rpc", type=str, choices=["server", "tracker"])
    parser.add_argument("--fcompile", type=str, choices=["ndk"])
    parser.add_argument("--port", type=int, default=9190)
    parser.add_argument("--check", action="store_true")
    parser.add_argument("--number", help="launches per timing", type=int, default=50)
    parser.add_argument("--perf_path", help="directory for the search's measured data and the learned models "
                        "(read by python -m flextensor_amd.train and by --use_model)", type=str, default="")
    parser.add_argument("--warm_up", help="warm-up epochs x points, e.g. 4x16", type=str, default="")
    parser.add_argument("--shapes", help="shape table to tune (driver specific)", type=str,
                        default="baseline")
    parser.add_argument("--cold", help="do not start from the shipped tuned log", action="store_true")


def run_driver(args, shapes, make_task, describe):
    """Common main of the three drivers: --test replays a log, --log tunes
    shapes[from_:to] and appends ``key:json`` lines."""
    import json
    import time
    from ..scheduler import schedule
    from ..utils import Config, RpcInfo
    rpc_info = RpcInfo(args.host, args.port, args.target_host, args.device_key, args.use_rpc,
                       args.fcompile, args.timeout)
    end = len(shapes) if args.to < 0 else args.to
    if args.test != "":
        with open(args.test, "r") as fin:
            for line in fin:
                if not line.strip() or line.startswith("#"):
                    continue
                name, string = line.split(":", 1)
                obj = json.loads(string)
                test(name, Config(obj[0], obj[1]), args.device, rpc_info=rpc_info,
                     check_result=args.check)
        return
    flog = open(args.log, "a") if args.log != "" else sys.stdout
    kwargs = {}
    if args.warm_up:
        a, b = args.warm_up.lower().split("x")
        kwargs["warm_up"] = (int(a), int(b))
    if getattr(args, "cold", False):
        kwargs["warm_start"] = False
    if getattr(args, "perf_path", ""):
        os.makedirs(args.perf_path, exist_ok=True)
        kwargs["perf_path"] = args.perf_path
    try:
        for i, shape in enumerate(shapes[args.from_:end]):
            print("Optimize %s shape %s [%.6f]" % (describe, str(shape), time.time()), flush=True)
            task, trials = make_task(i + args.from_, shape, args)
            beg = time.time()
            s, bufs, configs = schedule(
                task.key, slevel=args.slevel, rlevel=args.rlevel, op_trial=args.trials,
                timeout=args.timeout, op_stop=max(args.trials // 2, 1), method=args.method,
                use_model=args.use_model, parallel=args.parallel, rpc_info=rpc_info,
                number=args.number, force_inline=args.force_inline, trials=trials, **kwargs)
            endt = time.time()
            print("###################################### [%.6f]" % time.time())
            print("op schedules:")
            for config in configs.op_config_lst:
                print("----------------------------------")
                for name, value in config.items():
                    if value:
                        print(name, value)
            print("graph schedules:")
            for name, value in configs.graph_config.items():
                if value:
                    print(name, value)
            time_cost = evaluate(task.key, s, bufs, args.target, args.device, 100, rpc_info)
            # the log holds nothing but key:json lines, so the reference's readers
            # (line.split(":", 1) + json.loads on every line) take it as it is
            print(task.key + ":" + json.dumps(configs), file=flog, flush=True)
            print("Use", time_cost, "ms")
            print("Cost", endt - beg, "s")
            print()
    finally:
        if flog is not sys.stdout:
            flog.close()
