import os
import sys

import pytest

REPO_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if REPO_ROOT not in sys.path:
    sys.path.insert(0, REPO_ROOT)

import __graft_entry__ as entry  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    return entry.load_oracle()


@pytest.fixture(scope="session")
def nr_oracle():
    return entry.load_norm_rope_oracle()


@pytest.fixture(scope="session")
def dit_oracle():
    return entry.load_dit_attention_oracle()


@pytest.fixture(scope="session")
def block_oracle():
    return entry.load_dit_block_oracle()


@pytest.fixture(scope="session")
def net_oracle():
    return entry.load_dit_network_oracle()


@pytest.fixture(scope="session")
def pkg():
    """The package with its HIP library loaded; fails loudly when the library is not built."""
    return entry.load_package()


@pytest.fixture(scope="session")
def gpu():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


@pytest.fixture
def stream_override(pkg):
    """``stream_override(chunk=..., groups=...)`` steers short key sequences to (or away from) the query-streaming kernels through the
    library's own hook ``cosmos_attn_set_stream_override``; the library's choice is restored after the test."""
    lib = pkg._lib.load_library()

    def set_(chunk=0, groups=0):
        lib.cosmos_attn_set_stream_override(int(chunk), int(groups))

    yield set_
    lib.cosmos_attn_set_stream_override(0, 0)
