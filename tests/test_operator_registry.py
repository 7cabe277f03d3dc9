"""Registry rows of the ROCm inspection command against the generator's rules.

The reference validates its operator registry with tools/generate_operator_registry.py.  The
rules that a new row has to pass are restated here (syntax at :62-64, enumerations at :17-43,
admitted keys at :85-137, the per-operation checks at :424-597) and applied to the fragment
after the registry's operation defaults (config/operator/registry.json, "operation_defaults")
are laid under each row, as the generator does.  Where the reference tree is present the rows
are also merged into the real registry, read as JSON, to catch duplicate identities, paths and
unknown catalog names.
"""
import json
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FRAGMENT = os.path.join(ROOT, "clori_amd", "registry", "rocm_operator_rows.json")
REFERENCE_REGISTRY = "/root/reference/config/operator/registry.json"

IDENTIFIER = re.compile(r"^[a-z][a-z0-9]*(?:[._-][a-z0-9]+)*$")
FLAG = re.compile(r"^--[a-z0-9][a-z0-9-]*$")
WORD = re.compile(r"^[a-z0-9][a-z0-9._-]*$")
LANES = {"runtime-client", "offline-engine", "daemon-entrypoint", "REPL-local", "API-only", "test-only"}
VISIBILITIES = {"product-default", "product-advanced", "engineering", "automation", "API-only",
                "test-only", "removed"}
PLANES = {"Compile", "Run", "Execute", "Integrate", "Inspect", "System", "Profile"}
TTY_POLICIES = {"required", "optional", "forbidden"}
VALUE_TYPES = {"boolean", "u64", "number", "enum", "path", "name", "text", "delegated"}
REQUIREMENTS = {
    "daemon": {"absent", "optional", "required"},
    "model": {"none", "selected-config", "registry-model", "runtime-model"},
    "artifact": {"none", "descriptor", "admitted-artifact", "runtime-binding"},
    "backend": {"none", "optional", "required", "runtime"},
}
FORBIDDEN_TOP_LEVEL = {"dev", "eval", "evidence", "execute", "graph", "integrate", "quant", "system",
                       "tensor", "tokenizer"}
OPERATION_KEYS = {
    "CLI_projection", "TTY_policy", "adapter_argv", "adapter_id", "aliases", "architectural_plane",
    "arguments", "artifact_requirement", "backend_requirement", "command_path", "completion_provider",
    "daemon_requirement", "default_providers", "deprecation_state", "documentation_owner", "flag_sets",
    "flags", "input_schema", "lane", "model_requirement", "operation_id", "protocol_operation",
    "renderer_id", "result_schema", "schema_version", "side_effects", "slash_arguments",
    "slash_aliases", "slash_projection", "summary", "superseded_by", "test_owner", "validator_ids",
    "visibility",
}
ARGUMENT_KEYS = {"completion_provider", "enum_values", "multiplicity", "name", "range", "required",
                 "sensitive_display", "validator", "value_type"}
# config/operator/registry.json "operation_defaults"
OPERATION_DEFAULTS = {
    "CLI_projection": True, "TTY_policy": "optional", "adapter_argv": [], "aliases": [],
    "arguments": [], "artifact_requirement": "none", "backend_requirement": "none",
    "completion_provider": "none", "daemon_requirement": "absent", "default_providers": [],
    "deprecation_state": "current", "documentation_owner": "docs/operator-runbook.md",
    "flag_sets": [], "flags": [], "input_schema": "argv.v1", "model_requirement": "none",
    "protocol_operation": "none", "renderer_id": "human", "result_schema": "human.v1",
    "schema_version": 1, "side_effects": "read-only", "slash_projection": "none",
    "test_owner": "tests/client_cutover.sh", "validator_ids": ["syntax.delegated"],
}
# the catalog names the rows may refer to (config/operator/registry.json "catalogs")
VALIDATORS = {"syntax.delegated", "syntax.enum", "syntax.name", "syntax.none", "syntax.path",
              "syntax.text", "syntax.u64"}
RENDERERS = {"completion", "discovery", "human", "human-or-json", "none", "stream"}
COMPLETION_PROVIDERS = {"enum", "filesystem", "model-registry", "none", "session"}


def fragment():
    with open(FRAGMENT, encoding="utf-8") as stream:
        return json.load(stream)


def check_argument(argument):
    assert set(argument) <= ARGUMENT_KEYS
    assert argument["name"]
    assert argument.get("validator", "syntax.delegated") in VALIDATORS
    multiplicity = argument.get("multiplicity", "one")
    assert multiplicity in {"one", "optional", "many"}
    assert argument.get("completion_provider", "none") in COMPLETION_PROVIDERS
    value_type = argument.get("value_type", "text")
    assert value_type in VALUE_TYPES - {"boolean"}
    if value_type == "enum":
        assert argument.get("enum_values")
    assert argument.get("required", multiplicity == "one") == (multiplicity == "one")
    return multiplicity


def check_operation(raw, adapters, flag_sets):
    assert set(raw) <= OPERATION_KEYS
    operation = dict(OPERATION_DEFAULTS)
    operation.update(raw)
    assert IDENTIFIER.fullmatch(operation["operation_id"])
    assert operation["lane"] in LANES
    assert operation["visibility"] in VISIBILITIES
    assert operation["architectural_plane"] in PLANES
    path = operation["command_path"]
    assert path and all(WORD.fullmatch(word) for word in path)
    assert path[0] not in FORBIDDEN_TOP_LEVEL
    assert operation["adapter_id"] in adapters[operation["lane"]]
    assert not (operation["lane"] == "offline-engine" and operation["daemon_requirement"] == "required")
    assert operation["renderer_id"] in RENDERERS
    assert set(operation["validator_ids"]) <= VALIDATORS
    for name in operation["flag_sets"]:
        assert name in flag_sets
    seen_many = seen_optional = False
    for argument in operation["arguments"]:
        assert not seen_many
        multiplicity = check_argument(argument)
        seen_many |= multiplicity == "many"
        if multiplicity == "optional":
            seen_optional = True
        else:
            assert not (seen_optional and multiplicity == "one")
    for field in ("test_owner", "documentation_owner", "input_schema", "result_schema", "summary",
                  "side_effects"):
        assert isinstance(operation[field], str) and operation[field]
    if operation["CLI_projection"] and operation["visibility"] not in {"API-only", "test-only", "removed"}:
        assert operation["test_owner"] != "none" and operation["documentation_owner"] != "none"
    assert operation["TTY_policy"] in TTY_POLICIES
    for field, admitted in REQUIREMENTS.items():
        assert operation[f"{field}_requirement"] in admitted
    assert operation["slash_projection"] == "none" or operation["lane"] in {"runtime-client", "REPL-local"}
    assert all(isinstance(word, str) and word for word in operation["adapter_argv"])
    assert (operation["deprecation_state"] == "removed") == (operation["visibility"] == "removed")
    return operation


def test_fragment_uses_registry_keys_only():
    rows = fragment()
    assert rows["schema"] == "yvex.operator.registry.v1" and rows["schema_version"] == 1
    assert set(rows) <= {"catalogs", "operations", "schema", "schema_version"}
    assert set(rows["catalogs"]) == {"adapters"}
    assert set(rows["catalogs"]["adapters"]) <= {"runtime-client", "offline-engine",
                                                  "daemon-entrypoint", "REPL-local"}


def test_rows_pass_the_generator_rules():
    rows = fragment()
    adapters = {lane: set(names) for lane, names in rows["catalogs"]["adapters"].items()}
    for lane in ("runtime-client", "offline-engine", "daemon-entrypoint", "REPL-local"):
        adapters.setdefault(lane, set())
    identities, paths = set(), set()
    for raw in rows["operations"]:
        operation = check_operation(raw, adapters, flag_sets=set())
        assert operation["operation_id"] not in identities
        assert tuple(operation["command_path"]) not in paths
        identities.add(operation["operation_id"])
        paths.add(tuple(operation["command_path"]))
    assert "system.rocm" in identities and ("inspect", "rocm") in paths


def test_row_mirrors_the_cuda_row_shape():
    """system.rocm differs from system.cuda (config/operator/registry.json) only where it names
    the device runtime: adapter, argv, path, identity and the two texts."""
    row = next(o for o in fragment()["operations"] if o["operation_id"] == "system.rocm")
    assert row["adapter_id"] == "rocm" and row["adapter_argv"] == ["rocm-info"]
    assert row["architectural_plane"] == "System" and row["lane"] == "offline-engine"
    assert row["backend_requirement"] == "optional" and row["visibility"] == "product-default"
    assert row["arguments"] == [{"completion_provider": "none", "multiplicity": "many",
                                 "name": "arguments", "required": False,
                                 "validator": "syntax.delegated", "value_type": "text"}]


@pytest.mark.skipif(not os.path.exists(REFERENCE_REGISTRY), reason="reference tree not present")
def test_rows_merge_into_the_reference_registry():
    with open(REFERENCE_REGISTRY, encoding="utf-8") as stream:
        registry = json.load(stream)
    rows = fragment()
    assert registry["operation_defaults"] == OPERATION_DEFAULTS
    catalogs = registry["catalogs"]
    assert set(catalogs["validators"]) == VALIDATORS and set(catalogs["renderers"]) == RENDERERS
    assert set(catalogs["completion_providers"]) == COMPLETION_PROVIDERS
    adapters = {lane: set(names) for lane, names in catalogs["adapters"].items()}
    for lane, names in rows["catalogs"]["adapters"].items():
        assert not (adapters[lane] & set(names))          # the adapter names are new
        adapters[lane] |= set(names)
    identities = {o["operation_id"] for o in registry["operations"]}
    paths = {tuple(o.get("command_path", [])) for o in registry["operations"]}
    aliases = {tuple(a["path"]) for o in registry["operations"] for a in o.get("aliases", [])}
    cuda = next(o for o in registry["operations"] if o["operation_id"] == "system.cuda")
    for raw in rows["operations"]:
        operation = check_operation(raw, adapters, flag_sets=set(registry["flag_sets"]))
        assert operation["operation_id"] not in identities
        assert tuple(operation["command_path"]) not in paths | aliases
        assert set(raw) == set(cuda)                       # same fields as the CUDA row
    # `--backend rocm` rides on an existing plain value flag: no row changes for it
    attention = registry["flag_sets"]["cli_offline_graph_attention"]
    assert "--backend" in attention["values"] and FLAG.fullmatch("--backend")
