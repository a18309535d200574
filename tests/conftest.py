import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden_dir():
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def pytest_terminal_summary(terminalreporter):
    """Margins of the 16-bit parity bar over the cases of this run (gpu_util.MARGINS)."""
    gpu_util = sys.modules.get("gpu_util")
    margins = getattr(gpu_util, "MARGINS", None)
    if not margins:
        return
    terminalreporter.write_line("16-bit parity margins (worst row error / max|row|; row-floor coefficient the worst row needed):")
    for kind in ("out", "dq", "dk", "dv"):
        if kind in margins:
            rel, needed, rel_case, needed_case = margins[kind]
            terminalreporter.write_line(f"  {kind:>3}: {rel:.3e} [{rel_case}]   floor needed {max(needed, 0.0):.3e} [{needed_case}]")
    # the baseline configurations at full size, worst of their slices per tensor
    table = {}
    for name, rel, needed in getattr(gpu_util, "CASE_MARGINS", []):
        words = name.split()
        if words[0] == "full-size" and len(words) == 4:
            cell = table.setdefault(words[1], {}).setdefault(words[3], [0.0, 0.0])
            cell[0], cell[1] = max(cell[0], rel), max(cell[1], needed)
    for config, cells in table.items():
        terminalreporter.write_line(f"  {config}: " + "  ".join(f"{kind} {cells[kind][0]:.2e}/{cells[kind][1]:.2e}"
                                                                 for kind in ("out", "dq", "dk", "dv") if kind in cells))
