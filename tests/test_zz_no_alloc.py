"""The entry point that allocates nothing, ``velox_argmax_static``, called through ``ctypes`` and held against the
existing ``velox_argmax`` (which takes its scratch from the caller) and against ``torch.argmax``: two calls in a row,
the second with a smaller input, so that it runs over what the first left in the static array."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

_P, _I = ctypes.c_void_p, ctypes.c_int
MAX_PAIRS = 65536


@pytest.fixture(scope="module")
def core():
    from velox_amd.kernels import build

    lib = ctypes.CDLL(build.ensure_core())
    lib.velox_argmax.argtypes = [_P, _P, _P, _I, _I, _I, _P]
    lib.velox_argmax.restype = _I
    lib.velox_argmax_static.argtypes = [_P, _P, _I, _I, _I, _P]
    lib.velox_argmax_static.restype = _I
    lib.velox_argmax_static_init.argtypes = []
    lib.velox_argmax_static_init.restype = _I
    lib.velox_no_alloc_error_text.argtypes = [_I]
    lib.velox_no_alloc_error_text.restype = ctypes.c_char_p
    return lib


def _stream():
    return _P(torch.cuda.current_stream().cuda_stream)


def _logits(rows, vocab, seed):
    generator = torch.Generator(device="cpu").manual_seed(seed)
    logits = torch.randn((rows, vocab), generator=generator, dtype=torch.float32)
    # the largest value twice in some rows: the smaller index has to win, also across chunks
    for row in range(0, rows, 3):
        place = int(torch.randint(0, vocab - 1, (1,), generator=generator))
        logits[row, place] = 9.0
        logits[row, vocab - 1] = 9.0
    return logits.cuda()


def _existing(core, logits, chunks):
    rows, vocab = logits.shape
    out = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    partial = torch.empty((rows, chunks, 2), dtype=torch.int32, device="cuda")
    assert core.velox_argmax(_P(logits.data_ptr()), _P(out.data_ptr()), _P(partial.data_ptr()), rows, vocab, chunks, _stream()) == 0
    return out


def _static(core, logits, chunks):
    rows, vocab = logits.shape
    out = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    status = core.velox_argmax_static(_P(logits.data_ptr()), _P(out.data_ptr()), rows, vocab, chunks, _stream())
    assert status == 0, core.velox_no_alloc_error_text(status)
    return out


def test_static_argmax_matches_the_allocating_one_on_two_calls_in_a_row(core):
    assert core.velox_argmax_static_init() == 0
    for rows, vocab, chunks, seed in ((48, 152064 + 3, 10, 0), (5, 4099, 2, 1), (7, 1000, 1, 2), (64, 152064, 74, 3), (3, 320, 5, 4)):
        logits = _logits(rows, vocab, seed)
        got = _static(core, logits, chunks)
        want = _existing(core, logits, chunks)
        torch.cuda.synchronize()
        assert torch.equal(got, want), (rows, vocab, chunks)
        assert torch.equal(got.long(), torch.argmax(logits, dim=-1)), (rows, vocab, chunks)  # (torch takes the first of equal values too)


def test_static_argmax_allocates_nothing(core):
    logits = _logits(16, 32000, 5)
    out = torch.empty(16, dtype=torch.int32, device="cuda")
    assert core.velox_argmax_static_init() == 0
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        assert core.velox_argmax_static(_P(logits.data_ptr()), _P(out.data_ptr()), 16, 32000, 8, _stream()) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before
    assert torch.equal(out.long(), torch.argmax(logits, dim=-1))


def test_static_argmax_refuses_what_its_array_cannot_hold(core):
    rows, chunks = 300, 256  # 76,800 pairs
    assert rows * chunks > MAX_PAIRS
    logits = torch.zeros((rows, 4096), dtype=torch.float32, device="cuda")
    out = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    status = core.velox_argmax_static(_P(logits.data_ptr()), _P(out.data_ptr()), rows, 4096, chunks, _stream())
    assert status == -2
    assert b"65536" in core.velox_no_alloc_error_text(status)
    assert core.velox_argmax_static(_P(logits.data_ptr()), _P(out.data_ptr()), rows, 4096, 0, _stream()) == -1
    assert core.velox_argmax_static(_P(0), _P(out.data_ptr()), rows, 4096, 1, _stream()) == -1
    torch.cuda.synchronize()
    assert bool((out == -7).all())  # nothing was launched
    # the largest call that fits
    rows, chunks = 256, 256
    logits = _logits(rows, 8192, 6)
    assert torch.equal(_static(core, logits, chunks).long(), torch.argmax(logits, dim=-1))
