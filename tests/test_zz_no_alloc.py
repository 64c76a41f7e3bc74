"""The argmax entry point that allocates nothing (its partial results live in a device array inside the library),
called through ctypes as a caller without torch would, against the entry point with a workspace argument."""
import ctypes

import pytest
import torch

from alice_llm_amd.hip import ops

pytestmark = pytest.mark.gpu


def test_argmax_without_allocation_matches_argmax_with_a_workspace():
    ops.library()                                            # builds the library if it is not built
    lib = ctypes.CDLL(ops.library_path())
    lib.alice_argmax_static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.alice_argmax_static.restype = ctypes.c_int
    lib.alice_argmax_static_init.restype = ctypes.c_int
    lib.alice_last_error.restype = ctypes.c_char_p
    lib.alice_argmax_chunks.argtypes = [ctypes.c_int, ctypes.c_int]
    assert lib.alice_argmax_static_init() == 0, lib.alice_last_error()
    g = torch.Generator(device="cuda").manual_seed(3)
    stream = torch.cuda.current_stream().cuda_stream
    # two calls in a row on one stream, the second with a smaller input: it finds the first call's partial
    # results in the shared array and must not read them
    # (256 rows of 131,072 use the array to its last pair: 512 pairs is the most that the chunk rule asks for)
    for B, V in ((8, 256000), (3, 50000), (256, 131072), (64, 131072), (1, 1000), (300, 20000)):
        logits = torch.randn(B, V, generator=g, device="cuda")
        logits[0, V - 7] = 50.0                              # a maximum in the last chunk
        if B > 1:
            logits[1, 5] = logits[1, V // 2] = 60.0          # equal maxima: the lowest index wins
        want = ops.argmax(logits)
        out = torch.full((B,), -1, dtype=torch.int32, device="cuda")
        rc = lib.alice_argmax_static(logits.data_ptr(), out.data_ptr(), B, V, stream)
        assert rc == 0, lib.alice_last_error()
        torch.cuda.synchronize()
        assert B * lib.alice_argmax_chunks(B, V) <= 512 and (lib.alice_argmax_chunks(B, V) > 1 or V < 16384 or B > 256)
        assert torch.equal(out, want) and out[0] == V - 7 and (B == 1 or out[1] == 5)
    assert 256 * lib.alice_argmax_chunks(256, 131072) == 512
    # no size asks for more than the array holds (the chunk rule and the array share one constant), so the refusal
    # of too many pairs cannot be provoked from outside; a missing pointer is refused the same way, before any launch
    assert max(b * lib.alice_argmax_chunks(b, v) for b in (1, 2, 7, 64, 255, 256, 257, 512, 4096) for v in (16384, 1 << 20, 1 << 24)
               if lib.alice_argmax_chunks(b, v) > 1) <= 512
    out = torch.zeros(1, dtype=torch.int32, device="cuda")
    assert lib.alice_argmax_static(None, out.data_ptr(), 1, 100, stream) != 0
    assert b"logits" in lib.alice_last_error()
