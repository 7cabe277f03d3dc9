"""Binary layout of the structures that cross the backend boundary.

tests/abi/layout_probe.c prints sizeof/offsetof/enum values; it is compiled against
include/yvex_rocm.h and, when the reference tree is present, against the reference's own
headers (include/yvex/internal/transformer.h:245-339, include/yvex/internal/backend.h:143-290,
include/yvex/backend.h:13-140, include/yvex/core.h:13-48).  tests/abi/reference_layout.txt
holds the numbers the reference headers gave, so the check also runs without the tree.
"""
import ctypes as C
import os
import subprocess

import pytest

from clori_amd import binding as B

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROBE = os.path.join(ROOT, "tests", "abi", "layout_probe.c")
EXPECTED = open(os.path.join(ROOT, "tests", "abi", "reference_layout.txt")).read()
REFERENCE_INCLUDE = "/root/reference/include"


def run_probe(tmp_path, name, flags):
    exe = str(tmp_path / name)
    subprocess.check_call(["gcc", "-std=c11", "-D_POSIX_C_SOURCE=200809L", *flags, PROBE, "-o", exe])
    return subprocess.check_output([exe]).decode()


def test_header_layout_equals_the_reference_numbers(tmp_path):
    ours = run_probe(tmp_path, "ours", ["-I" + os.path.join(ROOT, "include")])
    assert ours == EXPECTED


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE_INCLUDE, "yvex")),
                    reason="reference tree not present")
def test_committed_numbers_are_what_the_reference_headers_give(tmp_path):
    ref = run_probe(tmp_path, "ref", ["-DPROBE_REFERENCE_HEADERS", "-I" + REFERENCE_INCLUDE])
    assert ref == EXPECTED


def expected(kind, name):
    for line in EXPECTED.splitlines():
        k, rest = line.split(" ", 1)
        label, value = rest.rsplit(" ", 1)
        if k == kind and label == name:
            return int(value)
    raise KeyError(name)


def test_ctypes_mirrors_have_the_same_layout():
    assert C.sizeof(B.Error) == expected("sizeof", "yvex_error")
    assert C.sizeof(B.OperationFacts) == expected("sizeof", "yvex_backend_operation_facts")
    assert C.sizeof(B.DeviceTensor) == expected("sizeof", "struct yvex_device_tensor")
    assert C.sizeof(B.AttentionRequirement) == expected("sizeof", "yvex_transformer_attention_requirement")
    assert C.sizeof(B.AttentionRequest) == expected("sizeof", "yvex_transformer_attention_request")
    assert C.sizeof(B.BandwidthEvidence) == expected("sizeof", "yvex_backend_bandwidth_evidence")
    assert C.sizeof(B.TransformerOperations) == expected("sizeof", "struct yvex_backend_transformer_operations")
    for member in ("attention_workspace_required", "attention_execute"):
        assert getattr(B.TransformerOperations, member).offset == expected(
            "offsetof", "struct yvex_backend_transformer_operations." + member)
