"""A plain device-to-device copy of known size, for calibrating HBM byte counters.

    rocprofv3 --pmc FETCH_SIZE --kernel-trace -- python3 -m llminfer_amd.hbm_calibration

copies a 1 GiB buffer a few times with an elementwise copy kernel: every dispatch reads 1 GiB and writes
1 GiB, far more than any cache holds, so counter / 2**30 per dispatch is the counter's scale factor.
"""
import sys

import torch

GIB = 1 << 30


def main(reps=6):
    if not torch.cuda.is_available():
        print("hbm_calibration: no GPU", file=sys.stderr)
        return 1
    src = torch.empty(GIB // 4, dtype=torch.float32, device="cuda")
    src.fill_(1.0)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    for _ in range(reps):
        dst.copy_(src)
    torch.cuda.synchronize()
    print("copied %d x %d bytes" % (reps, GIB))
    return 0


if __name__ == "__main__":
    sys.exit(main())
