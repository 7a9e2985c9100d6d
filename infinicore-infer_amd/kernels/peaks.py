"""What the device reaches at most, measured: the matrix cores' bfloat16 rate with nothing but MFMA instructions, a
read of memory that does nothing else, and a device-to-device copy.  The reports price kernels against the published
peaks (2.5 PFLOP/s, 8 TB/s); these are the figures a kernel can actually be compared with.

    python -m infinicore_infer_amd.kernels.peaks
"""
import sys

import torch

from .lib import check, get_lib


def _time(fn, reps: int) -> float:
    """Milliseconds per call, from events around `reps` calls."""
    fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


def mfma_bf16_tflops(iters: int = 20000, blocks_per_unit: int = 8) -> float:
    lib = get_lib()
    sink = torch.zeros(4, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    ops = [0]

    def run():
        ops[0] = lib.ic_peak_mfma_bf16(sink.data_ptr(), iters, blocks_per_unit, stream)
        if ops[0] < 0:
            check(int(ops[0]), "ic_peak_mfma_bf16")
    ms = _time(run, 5)
    return ops[0] / (ms * 1e-3) / 1e12


def read_tbs(megabytes: int = 4096, blocks_per_unit: int = 8) -> float:
    lib = get_lib()
    buf = torch.empty(megabytes << 20, dtype=torch.uint8, device="cuda").fill_(1)
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    ms = _time(lambda: check(lib.ic_peak_read(buf.data_ptr(), buf.numel(), blocks_per_unit, sink.data_ptr(), stream), "ic_peak_read"), 10)
    return buf.numel() / (ms * 1e-3) / 1e12


def copy_tbs(megabytes: int = 2048) -> float:
    """Bytes read plus bytes written per second of a device-to-device copy."""
    a = torch.empty(megabytes << 20, dtype=torch.uint8, device="cuda").fill_(1)
    b = torch.empty_like(a)
    ms = _time(lambda: b.copy_(a), 10)
    return 2 * a.numel() / (ms * 1e-3) / 1e12


def main(argv=None) -> int:
    if not torch.cuda.is_available():
        print("no GPU", file=sys.stderr)
        return 1
    print("device: %s, %d compute units" % (torch.cuda.get_device_name(0), torch.cuda.get_device_properties(0).multi_processor_count))
    for bpu in (4, 8):
        print("matrix cores, bfloat16, v_mfma_f32_32x32x16_bf16 only, %d blocks of 4 waves a unit: %.0f TFLOP/s" % (bpu, mfma_bf16_tflops(blocks_per_unit=bpu)))
    for bpu in (4, 8, 16):
        print("read of 4 GiB, 16-byte loads, %d blocks a unit: %.2f TB/s" % (bpu, read_tbs(blocks_per_unit=bpu)))
    print("device-to-device copy of 2 GiB (read + write): %.2f TB/s" % copy_tbs())
    return 0


if __name__ == "__main__":
    sys.exit(main())
