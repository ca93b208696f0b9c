"""Shared helpers of the GPU parity tests: inputs come from the oracle's generator (host) or
the library's generator (device, bit-identical for UNIFORM/GRID/SMALLINT), results are
compared with the oracle under the stated tolerance."""
import numpy as np

# fp16 result vs fp64 sum: |err| <= 2 ulp_fp16(result) + 1e-3 * sqrt(segment size)
ULPS = 2.0
ABS_PER_SQRT = 1e-3


def to_dev(x16):
    import torch

    return torch.from_numpy(np.ascontiguousarray(x16).view(np.float16)).cuda()


def to_host(t):
    import torch

    torch.cuda.synchronize()
    return t.detach().cpu().numpy().view(np.uint16)


def expect_ok(oracle, got16, ref64, seg, what):
    bad, worst, first = oracle.check_f16(got16, ref64, seg, ULPS, ABS_PER_SQRT)
    assert bad == 0, f"{what}: {bad} outside tolerance, worst excess {worst}, first at {first}"
