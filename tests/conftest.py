"""Test set-up: the repository root and this folder on the import path; tests marked ``gpu`` are skipped where
no GPU is visible (the marker itself is registered in pytest.ini); every test starts from random number generators
seeded with its own name, so what a test draws does not depend on which tests ran before it."""
import pathlib
import random
import sys
import zlib

import pytest

HERE = pathlib.Path(__file__).resolve().parent
for folder in (HERE, HERE.parent):
    if str(folder) not in sys.path:
        sys.path.insert(0, str(folder))

_gpu_visible = None


def pytest_runtest_setup(item):
    global _gpu_visible
    if item.get_closest_marker("gpu") is None:
        return
    if _gpu_visible is None:
        import torch

        _gpu_visible = torch.cuda.is_available()
    if not _gpu_visible:
        pytest.skip("needs a GPU")


@pytest.fixture(autouse=True)
def seeded_by_test_name(request):
    import torch

    seed = zlib.crc32(request.node.nodeid.encode())
    random.seed(seed)
    torch.manual_seed(seed)  # (the generators of every device)
