"""GPU: the exchange of split partials inside one XCC's L2 and what guards it.

The short-list kernel lets the split workgroups of a head row meet in their XCC's L2 when the
library's probe found that the device deals workgroups to XCCs round-robin and the grid puts all
splits of a row on one XCC.  The first launch on a hardware queue records the XCC the queue starts
at (and exchanges through memory); from then on every workgroup checks its own placement against
that record; one that disagrees computes its whole head row alone and marks the row, and from the
next launch on a marked row is computed by one workgroup.  TIDAL_XCC_LOCAL=twist makes the
workgroups 2 and 3 (mod 8) of every dispatch take themselves for misplaced, so that they take that
path without any workgroup being misplaced; TIDAL_XCC_LOCAL=0 switches the L2 exchange off.  Each setting runs in a child process
(the probe runs once per process).  Outputs are compared with the CPU oracle in every case (max-abs
2e-3 fp16 / 1e-2 bf16); semantics as kernels/include/decode/decode_attn.cuh:432-658 of the
reference."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


def _child(setting):
    env = dict(os.environ)
    if setting is None:
        env.pop("TIDAL_XCC_LOCAL", None)
    else:
        env["TIDAL_XCC_LOCAL"] = setting
    res = subprocess.run([sys.executable, os.path.join(HERE, "_xcc_child.py")], env=env, capture_output=True,
                         text=True, timeout=600)
    assert res.returncode == 0, res.stderr[-2000:]
    return json.loads(res.stdout.strip().splitlines()[-1])["cases"]


def test_partials_meet_in_l2_and_results_match(cuda):
    cases = _child(None)
    for c in cases:
        assert c["worst_error_over_tolerance"] <= 1.0, c
        assert c["marked_slots"] == [] and c["memory_tickets_nonzero"] == [] and c["l2_tickets_nonzero"] == [], c
    if not any("partials meet in L2" in k for c in cases for k in c["kernels"]):
        pytest.skip("the probe found no regular workgroup placement on this device: exchange through memory")
    for c in cases:
        assert all("partials meet in L2" in k for k in c["kernels"]), c


def test_switched_off(cuda):
    for c in _child("0"):
        assert c["worst_error_over_tolerance"] <= 1.0, c
        assert not any("L2" in k for k in c["kernels"]), c
        assert c["marked_slots"] == [] and c["memory_tickets_nonzero"] == [] and c["l2_tickets_nonzero"] == [], c


def test_misplaced_workgroups_compute_their_rows_alone(cuda):
    """The head rows 2, 3 (mod 8) hold workgroups that see "another XCC than the round-robin puts me
    on": results stay right in the launch where that happens and in
    every later one (other list lengths and plans on the same workspace included), exactly those
    rows' ticket slots are marked, no memory-side ticket is left behind, and the only L2-side tickets
    left behind belong to marked slots."""
    cases = _child("twist")
    if not any("partials meet in L2" in k for c in cases for k in c["kernels"]):
        pytest.skip("the probe found no regular workgroup placement on this device")
    for c in cases:
        assert c["worst_error_over_tolerance"] <= 1.0, c
        per_row = c["heads_per_row"]
        want = [r * per_row + j for r in range(c["rows"]) if r % 8 in (2, 3) for j in range(per_row)]
        assert c["marked_slots"] == want, c
        assert c["memory_tickets_nonzero"] == [], c
        assert set(c["l2_tickets_nonzero"]) <= set(want), c
