import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """Model folders (config.json + model.safetensors, random bf16 weights) of
    the tiny configurations, made once in a temporary folder."""
    from helpers import TINY, make_model_folder
    root = tmp_path_factory.mktemp("models")
    return {name: make_model_folder(str(root / name), name) for name in TINY}


@pytest.fixture(scope="session")
def sinepel_folders(tmp_path_factory):
    """Model folders of the small Sinepel configurations, made once in a temporary folder."""
    from sinepel_helpers import SMALL, make_folder
    root = tmp_path_factory.mktemp("sinepel")
    return {name: make_folder(str(root / name), name) for name in SMALL}


@pytest.fixture(scope="session")
def kapanex_folders(tmp_path_factory):
    """Model folders of the small Kapanex configurations, made once in a temporary folder."""
    from kapanex_helpers import SMALL, make_folder
    root = tmp_path_factory.mktemp("kapanex")
    return {name: make_folder(str(root / name), name) for name in SMALL}


@pytest.fixture(scope="session")
def kapanex_clear_folders(tmp_path_factory):
    """The same configurations with weights whose routers never have a close call (for comparisons in bfloat16)."""
    from kapanex_helpers import SMALL, make_folder
    root = tmp_path_factory.mktemp("kapanex_clear")
    return {name: make_folder(str(root / name), name, clear_routing=True) for name in SMALL}


@pytest.fixture(scope="session")
def gimipel_folders(tmp_path_factory):
    """Model folders of the small Gimipel configurations, made once in a temporary folder."""
    from gimipel_helpers import SMALL, make_folder
    root = tmp_path_factory.mktemp("gimipel")
    return {name: make_folder(str(root / name), name) for name in SMALL}


@pytest.fixture(scope="session")
def gimipel_clear_folders(tmp_path_factory):
    """The same configurations with weights whose routers read nothing that rounding touches and whose scores are
    of a size that a softmax does not multiply rounding with (for comparisons in bfloat16)."""
    from gimipel_helpers import SMALL, make_folder
    root = tmp_path_factory.mktemp("gimipel_clear")
    return {name: make_folder(str(root / name), name, clear_routing=True, mild=True) for name in SMALL}
