"""copy_rates.py -- what this GPU's memory side gives plain torch kernels, for scale: copy, fill and
sum at 64 MiB, 256 MiB and 1 GiB (the first fits the memory-side cache together with its destination).

    run: python3 copy_rates.py
"""
import torch

torch.cuda.init()
for mb in (64, 256, 1024):
    n = mb * 1024 * 1024 // 4
    a = torch.rand(n, device="cuda")
    b = torch.empty_like(a)
    for what, fn, nbytes in (("copy", lambda: b.copy_(a), 2 * n * 4), ("fill", lambda: b.fill_(1.0), n * 4),
                             ("sum", lambda: a.sum(), n * 4)):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(50):
            fn()
        e1.record()
        e1.synchronize()
        us = e0.elapsed_time(e1) / 50 * 1e3
        print("%-4s %4d MiB: %7.1f us  %5.2f TB/s" % (what, mb, us, nbytes / us / 1e6))
