import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    config.addinivalue_line("markers", "pack_auto: run once, with the library's own choice of packing ignored tokens "
                                       "(full-size cases, where that choice is to pack)")


def pytest_sessionstart(session):
    """Load what is built; compile the library only when there is none (hipcc cross-compiles without a GPU)."""
    from linear_cross_entropy_loss_amd import _lib

    if not _lib.LIB_PATH.exists():
        from linear_cross_entropy_loss_amd.build import build

        build(force=True)


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


ROUTE_MODULES = ("test_parity_gpu", "test_configs_gpu", "test_weight_layout_gpu")


def pytest_generate_tests(metafunc):
    # GPU tests run twice: with the tokens of ignored labels packed away before the tile kernels, and
    # without (by default the library chooses by problem size, which would leave small test shapes unpacked)
    if metafunc.definition.get_closest_marker("pack_auto") is not None:
        return
    if metafunc.definition.get_closest_marker("gpu") is not None and "pack_mode" in metafunc.fixturenames:
        metafunc.parametrize("pack_mode", ["pack", "nopack"], indirect=True)
    # The parity tests that go through autograd run on both routes: gradients from the forward's single evaluation
    # of the logits (the default where the problem allows it), and the loss-only forward with a backward that
    # recomputes the logit tiles.
    if (metafunc.definition.get_closest_marker("gpu") is not None and "route" in metafunc.fixturenames
            and metafunc.module.__name__ in ROUTE_MODULES):
        metafunc.parametrize("route", ["one_pass", "two_pass"], indirect=True)


@pytest.fixture(autouse=True)
def pack_mode(request):
    mode = getattr(request, "param", None)
    if mode is None:
        yield None
        return
    from linear_cross_entropy_loss_amd import _lib, ops

    token = ops.pack_rows.set(_lib.PACK_ALWAYS if mode == "pack" else _lib.PACK_NEVER)
    yield mode
    ops.pack_rows.reset(token)  # (also undoes whatever the test itself set in between)


@pytest.fixture(autouse=True)
def route(request):
    mode = getattr(request, "param", None)
    from linear_cross_entropy_loss_amd import ops

    if mode is None:
        token = ops.one_pass.set(True)
        yield None
        ops.one_pass.reset(token)  # (also undoes whatever the test itself set)
        return

    # (wherever the route fits the scratch bound, also on shapes so small that the library would not choose it)
    token = ops.one_pass.set("always" if mode == "one_pass" else False)
    yield mode
    ops.one_pass.reset(token)
