"""The reference's tuner caches as a coverage checklist for the code generator.

benchmark/**/tuner_cache.db of the reference hold one row per problem its tuner
ran: shape, operand layouts and the seven epilogue-node counts
(python/gtl/compiler/autotuner/tuner_base.py:107-152).  The keys are committed
as data (tests/golden/reference_tuner_keys.json, written by
tests/golden/make_reference_tuner_keys.py).  For every GEMM / BMM key a
synthetic epilogue with exactly those counts is traced behind a product of that
shape and layout, must land in one fused kernel whose own counts equal the
key's, its module must compile for gfx950, and the module's host side must
accept the problem at its real size (evt_workspace_bytes runs every range and
alignment check of the launch path; no kernel runs here).  The row-wise
anchors' keys are checked the same way against the softmax / layer norm
modules."""
import ctypes
import json
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

import pytest
import torch

from evt_ae_amd import jit
from evt_ae_amd.workloads import fused_nodes
from tests import patterns as W
from tests.util import fake_argument_block

FIXTURE = Path(__file__).resolve().parent / "golden" / "reference_tuner_keys.json"



def test_fixture_holds_the_reference_catalogue():
    doc = json.loads(FIXTURE.read_text())
    counts = {t: len(v) for t, v in doc["tables"].items()}
    assert counts == {"best_config_mm": 148, "best_config_bmm": 21, "best_config_softmax": 20,
                      "best_config_softmax_backward": 4, "best_config_layernorm": 8,
                      "best_config_layernorm_backward": 8}
    assert len(doc["files"]) == 10
    # the problems the path's limits are tested on are among them
    mm = doc["tables"]["best_config_mm"]
    for key in ("2048_670208_512_h_h_R_C_1_1_0_1_1_0_0", "736389_64_128_h_h_R_C_0_1_0_1_0_0_0",
                "16384_1024_30528_h_h_R_R_1_0_2_1_2_0_0", "64_64_736389_h_h_C_R_0_0_0_1_0_0_0",
                "33792_768_768_h_h_R_C_0_1_0_1_0_0_0"):
        assert key in mm, key
    assert "512_512_512_64_h_h_R_R_0_1_0_1_0_0_1" in doc["tables"]["best_config_bmm"]


def _lower_all():
    ops = []
    for table, key, case in W.reference_key_cases():
        mod, metas = W.counted_epilogue(case)
        gm = W.fuse(mod, metas)
        nodes = fused_nodes(gm)
        assert len(nodes) == 1, (key, len(nodes))
        ops.append((key, case, gm, nodes[0].target))
    return ops


@pytest.fixture(scope="module")
def lowered():
    return _lower_all()


def test_every_gemm_key_lands_in_one_fused_kernel_with_the_keys_counts(lowered):
    assert len(lowered) == 148 + 21
    for key, case, gm, op in lowered:
        want = case["counts"] or (0, 0, 0, 1, 0, 0, 0)      # first-stage keys: a plain store
        got = op.ir.epilogue_counts()
        assert tuple(got) == tuple(want), (key, got)
        M, N, K, L = op.problem
        assert (M, N, K, L) == (case["M"], case["N"], case["K"], case["L"]), key
        # operand layouts as the key says (R: [M, K] / [K, N] row-major)
        assert op.a_kc == case["a_row"] and op.b_kc == (not case["b_row"]), key
        if want[6]:
            # a value of the [N] vectors alone that the epilogue uses and other kernels read (the reference's
            # VisitorRowStore): computed and written by the fused kernel, nothing of it is left in the graph
            assert not any(n.op == "call_function" and n.target in (torch.ops.aten.mul, torch.ops.aten.rsub)
                           for n in gm.graph.nodes), key


def test_every_gemm_key_builds_and_accepts_its_problem_size(lowered):
    modules = {}
    for key, case, gm, op in lowered:
        modules.setdefault(str(op.module.path), op.module)
    assert len(modules) >= 40            # distinct (epilogue structure, layout, tile) combinations
    with ThreadPoolExecutor(8) as pool:
        list(pool.map(lambda m: m.build(), modules.values()))
    for key, case, gm, op in lowered:
        km = op.module.ensure()
        assert km.lib.evt_abi_version() == jit.EVT_ABI_VERSION
        a = fake_argument_block(op)
        need = km.lib.evt_workspace_bytes(ctypes.byref(a))
        assert need >= 0, (key, need)
        want = case["counts"] or (0, 0, 0, 1, 0, 0, 0)
        tiles_m, tiles_n = -(-a.M // op.tile.bm), -(-a.N // op.tile.bn)
        spans = (want[4] and tiles_m > 1) or (want[5] and tiles_n > 1)
        assert (need > 0) == bool(spans) or need > 0, (key, need)      # reductions over several tiles need partials


def test_every_row_anchor_key_has_a_module_that_holds_its_rows():
    """(rows, columns) of the reference's softmax / layer norm tuner rows: the bare anchor traced at that shape
    picks a register-cached kernel that holds the row, and its host side accepts the problem."""
    doc = json.loads(FIXTURE.read_text())
    assert sum(len(doc["tables"][t]) for t in doc["tables"] if "mm" not in t) == 40
    ops = []
    for key, anchor, rows, cols, mod, metas in W.reference_row_key_cases():
        gm = W.fuse(mod, metas)
        (node,) = fused_nodes(gm)
        op = node.target
        assert op.row_spec.max_n >= cols, key
        assert op.problem[0] * op.problem[3] == rows and op.problem[1] == cols, (key, op.problem)
        ops.append((key, op))
    assert len(ops) == 18            # distinct (anchor, rows, columns)
    modules = {str(op.module.path): op.module for _, op in ops}
    with ThreadPoolExecutor(8) as pool:
        list(pool.map(lambda m: m.build(), modules.values()))
    for key, op in ops:
        a = fake_argument_block(op)
        assert op.module.ensure().lib.evt_workspace_bytes(ctypes.byref(a)) == 0, key
