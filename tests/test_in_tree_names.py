"""The ROCm arm against the reference's own backend object (skipped without the tree).

In the reference tree the arm is compiled against src/backend/private.h instead of the reduced
mirror in clori_amd/csrc/host/private.h.  That works only if every member of struct
yvex_backend the arm touches, and every slot of the vtable it fills, exists there under the same
name with a compatible type.  This test reads both headers and the arm's sources and checks
exactly that, member by member and slot by slot."""
import glob
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "clori_amd", "csrc", "host")
REFERENCE_PRIVATE = "/root/reference/src/backend/private.h"

pytestmark = pytest.mark.skipif(not os.path.exists(REFERENCE_PRIVATE),
                                reason="the reference tree is not present")


def strip_comments(text):
    return re.sub(r"/\*.*?\*/", " ", text, flags=re.S)


def struct_body(text, opener):
    start = text.index(opener)
    depth, at = 0, text.index("{", start)
    for i in range(at, len(text)):
        depth += text[i] == "{"
        depth -= text[i] == "}"
        if depth == 0:
            return text[at + 1:i]
    raise AssertionError(opener)


def backend_members(text):
    """name -> declaration text of every member of struct yvex_backend."""
    body = struct_body(strip_comments(text), "struct yvex_backend {")
    members = {}
    for statement in body.split(";"):
        statement = " ".join(statement.split())
        if not statement:
            continue
        head = statement.split(",")[0]
        kind = head[:head.rstrip().rfind(" ")].replace(" *", "*").strip() if " " in head else ""
        for piece in statement.split(","):
            name = re.findall(r"[A-Za-z_][A-Za-z0-9_]*", piece)[-1]
            stars = piece.count("*")
            array = "[" in piece
            members[name] = (re.sub(r"\s+", " ", kind.replace("*", "")).strip(), stars, array)
    return members


def vtable_slots(text):
    body = struct_body(strip_comments(text), "typedef struct yvex_backend_vtable {")
    return {name: " ".join(decl.split())
            for decl in body.split(";") if decl.strip()
            for name in re.findall(r"\(\*\s*([A-Za-z_][A-Za-z0-9_]*)\s*\)", decl)[:1]}


def normalise(declaration):
    return re.sub(r"\s+", "", declaration).replace("structyvex_backend", "yvex_backend")


def test_every_backend_member_the_arm_touches_exists_in_the_reference_object():
    ours = backend_members(open(os.path.join(HOST, "private.h")).read())
    theirs = backend_members(open(REFERENCE_PRIVATE).read())
    used = set()
    for path in glob.glob(os.path.join(HOST, "*.c")) + glob.glob(os.path.join(HOST, "*.h")):
        text = strip_comments(open(path).read())
        used |= set(re.findall(r"(?:backend|owner|context_owner|executor|\)\s*)->\s*([A-Za-z_][A-Za-z0-9_]*)", text))
    touched = sorted(name for name in ours if name in used)
    assert {"kind", "status", "vtable", "stats", "impl", "lifecycle", "resource_owner",
            "workspace_cursor", "tensor_id_next", "virtual_tensor_ready"} <= set(touched)
    for name in ours:                       # the mirror declares nothing the reference lacks
        assert name in theirs, "struct yvex_backend of the reference has no member " + name
        assert ours[name] == theirs[name], (name, ours[name], theirs[name])


def test_every_vtable_slot_the_arm_fills_exists_in_the_reference_table():
    ours = vtable_slots(open(os.path.join(HOST, "private.h")).read())
    theirs = vtable_slots(open(REFERENCE_PRIVATE).read())
    filled = set(re.findall(r"^\s*\.([a-z_]+)\s*=", open(os.path.join(HOST, "rocm_backend.c")).read(), re.M))
    assert filled and filled <= set(ours)
    for name, declaration in ours.items():
        assert name in theirs, "the reference vtable has no slot " + name
        assert normalise(declaration) == normalise(theirs[name]), name
    # operations without a reference counterpart are not a slot: the arm's own getter
    assert "rocm_attention_operations" not in ours


IN_TREE_SOURCES = ("rocm_attention.c", "rocm_backend.c", "rocm_capability.c", "rocm_driver.c",
                   "rocm_elementwise.c", "rocm_schedule.c", "rocm_virtual.c")


@pytest.mark.parametrize("source", IN_TREE_SOURCES)
def test_the_arm_compiles_against_the_reference_headers(source):
    """Every file of the ROCm arm goes through the compiler's front end as it would inside the
    reference tree: YVEX_ROCM_IN_TREE makes clori_amd/csrc/host/private.h include the tree's
    src/backend/private.h (the tree's struct yvex_backend, its vtable and its helpers) in place
    of the local mirror, and makes include/yvex_rocm.h take every mirrored type from the tree's
    public and internal headers.  Types, members, vtable slots and the prototypes of every
    function both sides declare are held against each other by the compiler, warnings are
    errors; nothing is linked and the reference's build system is not run."""
    import shutil
    import subprocess
    if not os.path.isdir("/opt/rocm/include/hip"):
        pytest.skip("the HIP headers the driver table is declared from are not installed")
    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    command = ["gcc", "-std=c11", "-fsyntax-only", "-Wall", "-Wextra", "-Wno-unused-parameter",
               "-Werror", "-DYVEX_ROCM_IN_TREE", "-D__HIP_PLATFORM_AMD__",
               "-I", os.path.join(ROOT, "include"), "-I", "/root/reference",
               "-I", "/root/reference/include", "-I", "/opt/rocm/include", "-I", HOST,
               "-I", os.path.dirname(HOST), os.path.join(HOST, source)]
    done = subprocess.run(command, capture_output=True, text=True)
    assert done.returncode == 0, done.stderr[-3000:]
    # and it is the tree's backend object that was compiled against, not the mirror
    seen = subprocess.run(["-E" if part == "-fsyntax-only" else part for part in command],
                          capture_output=True, text=True)
    assert seen.returncode == 0 and "resident_map_readonly" in seen.stdout
