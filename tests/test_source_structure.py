"""The structural limits the reference sets for its C sources (config/c_policy.json:15-28,
enforced there by tests/c_structure.py), held against this arm's host code, headers and
kernels: translation units of at most 2000 lines, headers of at most 600, functions of at
most 200 (one device function is longer and is named below), lines of at most 120
characters.  The warning set the reference requires of C sources
(config/c_policy.json:41-49) is the one the host objects are built with."""
import glob
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "clori_amd", "csrc")

TRANSLATION_UNIT_LINES = 2000
HEADER_LINES = 600
FUNCTION_LINES = 200
HARD_LINE_WIDTH = 120
REQUIRED_C_WARNINGS = ("-Wstrict-prototypes", "-Wmissing-prototypes", "-Wmissing-declarations",
                       "-Wshadow", "-Wformat=2", "-Wundef", "-Wvla")


def sources():
    found = []
    for pattern in ("host/*.c", "host/*.h", "host/*.hip", "kernels/*.hip", "kernels/*.h", "*.h",
                    "cli/*.c"):
        found += glob.glob(os.path.join(CSRC, pattern))
    found += glob.glob(os.path.join(ROOT, "include", "*.h"))
    found += glob.glob(os.path.join(ROOT, "oracle", "*.[ch]"))
    assert len(found) > 30
    return sorted(found)


def lines_of(path):
    with open(path) as fp:
        return fp.read().split("\n")


def test_file_lengths():
    for path in sources():
        limit = HEADER_LINES if path.endswith(".h") else TRANSLATION_UNIT_LINES
        assert len(lines_of(path)) <= limit, path


def test_line_widths():
    for path in sources():
        for number, line in enumerate(lines_of(path), 1):
            assert len(line) <= HARD_LINE_WIDTH, "%s:%d" % (path, number)


# The device function that holds one software pipeline in registers from its first line to
# its last (the statistics, accumulators and prefetched operands live in locals that the
# lambdas of the function share) and is longer than the limit: (file, first line of the
# function's text).  Everything else, host and device, is within it.
LONGER_DEVICE_FUNCTIONS = (
    ("mla.hip", "__device__ __forceinline__ void mla_decode("),
)


def test_function_lengths():
    # the sources keep the braces of a function body in column 0, and nothing else there
    longer = []
    for path in sources():
        lines = lines_of(path)
        opened = None
        for number, line in enumerate(lines, 1):
            if line == "{":
                opened = number
            elif line == "}" and opened is not None:
                if number - opened + 1 > FUNCTION_LINES:
                    head = opened - 2
                    starts = ("__device__", "static", "int ", "void ")
                    while head > 0 and not lines[head].startswith(starts):
                        head -= 1
                    longer.append((os.path.basename(path), lines[head]))
                opened = None
    for name, head in longer:
        assert any(name == n and head.startswith(h)
                   for n, h in LONGER_DEVICE_FUNCTIONS), (name, head)
    assert len(longer) == len(LONGER_DEVICE_FUNCTIONS)


def test_host_objects_are_built_with_the_required_warnings():
    makefile = open(os.path.join(CSRC, "Makefile")).read()
    flags = makefile[makefile.index("CFLAGS :="):makefile.index("HIPFLAGS :=")]
    for warning in REQUIRED_C_WARNINGS:
        assert warning in flags, warning


def test_exported_symbols_follow_the_reference_namespace():
    # config/c_policy.json:108-113: public symbols carry the yvex_ prefix and none of the
    # fragments that mark test, fixture, rendering or family code
    import subprocess
    library = os.path.join(ROOT, "clori_amd", "libyvex_rocm.so")
    listing = subprocess.run(["nm", "-D", "--defined-only", library], check=True,
                             capture_output=True, text=True).stdout
    names = [line.split()[-1] for line in listing.splitlines() if line.strip()]
    assert len(names) > 40
    for name in names:
        assert name.startswith("yvex_"), name
        for fragment in ("_fixture_", "_reference_", "_test_", "_render_", "_deepseek_"):
            assert fragment not in name, name
