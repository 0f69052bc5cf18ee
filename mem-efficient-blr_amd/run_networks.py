"""python run_networks.py --network dit_xl --methods blast dense  (cf. reference run_networks.py:4-13)."""
import argparse
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)

from network import METHODS, Network   # noqa: E402


def main():
    ap = argparse.ArgumentParser(description="Time a whole network with its linears replaced.")
    ap.add_argument("--network", required=True, choices=["dit_xl"])
    ap.add_argument("--methods", nargs="+", default=METHODS)
    args = ap.parse_args()
    n = Network(os.path.join(HERE, "configs", "networks", f"{args.network}.yaml"))
    n.benchmark(args.methods)
    n.summary()


if __name__ == "__main__":
    main()
