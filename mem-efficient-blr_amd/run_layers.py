"""python run_layers.py --device MI355X --network llama7b --layer gate_up_proj  (cf. reference run_layers.py:7-36)."""
import argparse
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)

from device import Device            # noqa: E402
from layer import Layer              # noqa: E402
from roofline import plot_roofline   # noqa: E402


def main():
    ap = argparse.ArgumentParser(description="Benchmark, verify and roofline one layer.")
    ap.add_argument("--device", required=True, help="Device name (e.g. MI355X)")
    ap.add_argument("--network", required=True, help="Network name (e.g. llama7b)")
    ap.add_argument("--layer", required=True, help="Layer name (e.g. gate_up_proj)")
    ap.add_argument("--num-seq", type=int, default=None, help="override num_seq of the YAML")
    args = ap.parse_args()
    d = Device(args.device)
    print(d)
    l = Layer(os.path.join(HERE, "configs", "layers", f"{args.network}.{args.layer}.yaml"))
    if args.num_seq:
        l.num_seq = args.num_seq
    print(l)
    out_dir = f"output/{args.network}/{args.layer}"
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "device_summary.txt"), "w") as f:
        f.write(repr(d))
    with open(os.path.join(out_dir, "layer_summary.txt"), "w") as f:
        f.write(repr(l))
    l.benchmark("all")
    l.verify("all")
    l.summary()
    plot_roofline(l, d, l.measured_ms())


if __name__ == "__main__":
    main()
