"""The committed known-answer vectors against the oracle and against the
product's host helpers."""
import json
import os

from flashoverlap_amd import tiling
from oracle import fo_oracle as O

KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "tiling_known_answers.json")))


def test_oracle_reproduces_the_known_answers():
    for c in KAT["reorder_indices"]:
        assert O.reorder_indices(c["S"], c["hint"]).tolist() == c["RA"]
        assert O.reorder_indices_literal(c["S"], c["hint"]) == c["RA"]
    for c in KAT["uniform_cseg"]:
        assert O.uniform_cseg(c["T"], c["w"]) == c["cSeg"]
    for c in KAT["compositions"]:
        assert O.compositions(c["n"]) == c["out"]
    for c in KAT["cseg_from_composition"]:
        assert O.cseg_from_composition(c["gp"], c["W"], c["T"]) == c["cSeg"]
    for c in KAT["group_of_slot"]:
        n = len(c["groups"])
        assert [O.group_of_slot_literal(c["cSeg"], s) for s in range(n)] == c["groups"]
        assert O.group_of_slots(c["cSeg"], range(n)).tolist() == c["groups"]
    for c in KAT["row_remap"]:
        args = (c["M"], c["N"], c["BM"], c["BN"], c["cSeg"], c["ws"])
        assert O.row_remap(*args).tolist() == c["RE"]
        assert O.row_remap_literal(*args) == c["RE"]


def test_host_helpers_reproduce_the_known_answers():
    for c in KAT["reorder_indices"]:
        assert tiling.reorder_indices(c["S"], c["hint"]).tolist() == c["RA"]
    for c in KAT["uniform_cseg"]:
        assert tiling.uniform_cseg(c["T"], c["w"]) == c["cSeg"]
    for c in KAT["compositions"]:
        assert tiling.integer_partitions(c["n"]) == c["out"]
    for c in KAT["cseg_from_composition"]:
        assert tiling.cseg_from_groups(c["gp"], c["W"], c["T"]) == c["cSeg"]
    for c in KAT["row_remap"]:
        assert tiling.generate_row_remap_array(c["M"], c["N"], c["BM"], c["BN"], c["cSeg"], c["ws"]).tolist() == c["RE"]
