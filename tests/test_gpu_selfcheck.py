"""The library's check of its own arithmetic short cuts, run on the card over every input there is: det_silu against
gate / (1 + det_expf(-gate)) for all 2^32 float32 gates (det_sigmoid likewise against 1 / (1 + det_expf(-score))), and the quantizer by the card's FP8 conversions
(quantize_codes4) against the quantizer's defining arithmetic (source/kernel_activation_quantize.cuh:52-133 of the
reference, which tests/test_gpu_linear.py holds byte for byte to the CPU oracle) for all 2^16 bfloat16 values under
all 2^8 scale codes. A disagreement names its first input."""
import ctypes as C
import struct
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("check,what", [(0, "det_silu over all float32"), (1, "quantize_codes4 over all values and scale codes"),
                                        (2, "det_sigmoid over all float32"), (3, "linear_silu within 2^-17 of det_silu over all float32")])
def test_short_cuts_equal_their_definitions(check, what):
    import anemone_amd as amd
    print("selfcheck", check, what, flush=True)
    sys.stdout.flush()
    amd.probe_library()
    card = amd.Card(64 << 20)
    try:
        blocks, threads = 4096, 256
        output = card.reserve(blocks * threads * 8, 256)
        card.upload(output, np.full(blocks * threads * 2, 0xFFFFFFFF, dtype=np.uint32))
        launch = amd.launches_of(1)
        launch[0].kernel = card.kernel("kernel_selfcheck", "arithmetic_selfcheck", 16)
        launch[0].grid[0], launch[0].grid[1], launch[0].grid[2] = blocks, 1, 1
        launch[0].block[0], launch[0].block[1], launch[0].block[2] = threads, 1, 1
        launch[0].argument_byte_count = 16
        record = struct.pack("<QII", output, check, 0)
        C.memmove(launch[0].argument, record, 16)
        card.run(launch)
        result = card.download(output, blocks * threads * 8, np.uint32).reshape(-1, 2)
        bad = np.flatnonzero(result[:, 0])
        assert bad.size == 0, "%d disagreements, the first at input 0x%08X" % (int(result[:, 0].sum()), int(result[bad[0], 1]))
    finally:
        card.close()
