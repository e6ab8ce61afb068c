"""Secondary bench workloads (LSTM, Swin) selected with bench.py --workload."""
import sys


def run(args):
    print("unknown workload %r" % args.workload, file=sys.stderr)
    sys.exit(2)
