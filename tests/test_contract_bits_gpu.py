"""The stored output bits of each arithmetic contract id (tests/golden/contract_bits.json, written by
tests/golden/make_contract_bits.py on an MI355X): a build whose kernels produce other bits for the
same id fails here."""

from __future__ import annotations

import importlib.util
import json
from pathlib import Path

import pytest

GOLDEN = Path(__file__).parent / "golden"


def _generator():
    spec = importlib.util.spec_from_file_location("make_contract_bits", GOLDEN / "make_contract_bits.py")
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


@pytest.mark.gpu
def test_kernels_reproduce_the_stored_bits_of_their_contract_ids():
    stored = json.loads((GOLDEN / "contract_bits.json").read_text())
    assert _generator().contract_bits() == stored


def test_stored_k_tree_bits_are_the_oracle_bits(oracle):
    # The k-tree contract is fully specified, so the GPU's stored bits must be the CPU oracle's.
    import hashlib

    import inputs

    stored = json.loads((GOLDEN / "contract_bits.json").read_text())
    a, b = inputs.config1()
    want = oracle.k_tree_gemm(inputs.bits(a), inputs.bits(b.t().contiguous()))
    assert hashlib.sha256(want.tobytes()).hexdigest() == stored["rlkernel.det_gemm.hip_ktree32_gfx950.v1"]["config1_det_gemm"]


def test_stored_sequential_chain_bits_are_the_oracle_bits(oracle):
    # Fully specified as well: one fp32 fused multiply-add per k, ascending.
    import hashlib

    import inputs

    stored = json.loads((GOLDEN / "contract_bits.json").read_text())
    a, b = inputs.config1()
    want = oracle.det_gemm_seq_f32(a.float().numpy(), b.t().contiguous().float().numpy())
    assert hashlib.sha256(want.tobytes()).hexdigest() == stored["rlkernel.det_gemm.hip_seqfma32_gfx950.v1"]["config1_det_gemm_fp32"]
