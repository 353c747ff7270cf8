import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def golden_names():
    with open(os.path.join(GOLDEN_DIR, "INDEX.txt")) as handle:
        return [line.strip() for line in handle if line.strip()]


class Golden:
    """One reference-written fixture: input, container buffers, symbol planes and dense output."""

    BUFFER_NAMES = ("payload", "offsets", "states", "stream_meta", "freq_tables", "scales", "layout")
    _UNSIGNED = {"payload": np.uint16, "offsets": np.uint32, "states": np.uint32, "freq_tables": np.uint16}

    def __init__(self, name):
        self.name = name
        data = np.load(os.path.join(GOLDEN_DIR, name + ".npz"), allow_pickle=False)
        self.dtype = str(data["dtype"])
        self.shape = tuple(int(v) for v in data["shape"])
        self.options = {str(k): float(v) for k, v in zip(data["options_keys"], data["options_values"])}
        self.actual_bpp = float(data["actual_bpp"])
        self.weight_bits = data["weight_bits"]
        self.restored_bits = data["restored_bits"]
        self.quant_state = data["quant_state"]
        self.cosets = data["cosets"].astype(np.int64)
        self.fields = data["fields"].astype(np.int64)
        self.buffers = {}
        for key in self.BUFFER_NAMES:
            value = data["buf_" + key]
            if key in self._UNSIGNED:      # stored as same-width signed bit patterns
                value = value.view(self._UNSIGNED[key])
            self.buffers[key] = value

    @property
    def config_kwargs(self):
        out = {}
        for key, value in self.options.items():
            out[key] = int(value) if key in ("tile_elements", "prob_bits", "row_rdo_iterations", "row_rdo_candidates") else value
        return out


@pytest.fixture(params=golden_names())
def golden(request):
    return Golden(request.param)
