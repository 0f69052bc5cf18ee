"""Device peaks for the roofline model (role of the reference's device.py:1-24, plus MI355X)."""


class Device:
    # name -> (memory bandwidth in B/s, peak dense fp16/bf16 matrix throughput in FLOP/s)
    KNOWN = {
        "MI355X": (8.0e12, 2.5166e15),                       # HBM3E 8 TB/s, dense fp16/bf16 MFMA
        "A40": (696 * 2**30, 149.7e12),                      # reference device.py:6-7
        "Jetson Orin Nano 8GB": (68.29 * 2**30, 10e12),      # reference device.py:9-10
    }

    def __init__(self, name):
        if name not in self.KNOWN:
            raise ValueError("Name not supported in Device class")
        self.name = name
        self.memory_bandwidth, self.peak_performance = self.KNOWN[name]
        self.break_point = self.peak_performance / self.memory_bandwidth

    def __repr__(self):
        bar = "-" * 30
        return (f"\n{'=' * 30}\nDevice Information:\n{bar}\n"
                f" Name               : {self.name}\n"
                f" Memory Bandwidth   : {self.memory_bandwidth / 2**30:.2f} GiB/s\n"
                f" Peak Performance   : {self.peak_performance / 1e12:.2f} TFLOP/s\n"
                f" Break Point        : {self.break_point:.2e} FLOPs/Byte\n{bar}")
