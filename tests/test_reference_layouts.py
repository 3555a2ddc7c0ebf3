"""The structures include/yvex_rocm.h mirrors from the reference must have the reference's layout:
a caller compiled against the reference's headers hands them to this library as they are.

For every mirrored structure and enumeration of the header, sizes, field offsets, field sizes and
enumerator values are printed by two programs, one compiled against include/yvex_rocm.h and one
against the reference's own headers (read where they lie, when they are present), and compared.
Types that exist only in this library (yvex_rocm_*) are not mirrored and are skipped; the few
members this library adds to a mirrored type are listed in ADDITIONS and must stay at the end
of their type so that the reference's members keep their places.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "yvex_rocm.h")
REFERENCE = "/root/reference"
REFERENCE_HEADERS = ["yvex/core.h", "yvex/backend.h", "yvex/gguf.h", "yvex/qtype.h", "yvex/internal/backend.h",
                     "yvex/internal/execution.h", "yvex/internal/execution_batch.h", "yvex/internal/moe.h",
                     "yvex/internal/quant_numeric.h", "yvex/internal/graph.h"]

# Members this library adds to a mirrored type (each justified where the header declares it).
ADDITIONS = {
    "YVEX_MOE_SCORING_SIGMOID",          # sigmoid scoring of the benchmark layer
}
# Declared for this library alone, or the reference's type under the library's own name.
OWN_TYPES = re.compile(r"^yvex_rocm_")
RENAMED = {"yvex_rocm_operation_facts": "yvex_backend_cuda_operation_facts",
           "yvex_rocm_moe_operations": "yvex_backend_moe_operations"}
ADAPTER = os.path.join(ROOT, "yvex_amd", "csrc", "reference_binding", "rocm_adapter.c")


def parse_header():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    structs, enums = {}, {}
    found = re.findall(r"typedef\s+struct\s*\w*\s*\{(.*?)\}\s*(\w+)\s*;", text, flags=re.S)
    # `struct name { ... };` whose typedef stands apart
    found += [(body, name) for name, body in re.findall(r"^struct\s+(\w+)\s*\{(.*?)\}\s*;", text,
                                                        flags=re.S | re.M)]
    for body, name in found:
        fields = []
        for statement in body.split(";"):
            statement = " ".join(statement.split())
            if not statement:
                continue
            pointer = re.search(r"\(\s*\*\s*(\w+)\s*\)\s*\(", statement)      # function pointer member
            if pointer:
                fields.append(pointer.group(1))
                continue
            for part in statement.split(","):
                member = re.search(r"(\w+)\s*(\[[^\]]*\])*\s*$", part.strip())
                if member:
                    fields.append(member.group(1))
        structs[name] = fields
    for body, name in re.findall(r"typedef\s+enum\s*\w*\s*\{(.*?)\}\s*(\w+)\s*;", text, flags=re.S):
        enums[name] = [e.split("=")[0].strip() for e in body.split(",") if e.strip()]
    return structs, enums


def program(includes, structs, enums):
    lines = ["#include <stddef.h>", "#include <stdio.h>"] + [f"#include {i}" for i in includes]
    lines.append("int main(void) {")
    for name, fields in structs.items():
        lines.append(f'    printf("{name} %zu\\n", sizeof({name}));')
        for field in fields:
            lines.append(f'    printf("{name}.{field} %zu %zu\\n", offsetof({name}, {field}), '
                         f"sizeof((({name} *)0)->{field}));")
    for name, members in enums.items():
        lines.append(f'    printf("{name} %zu\\n", sizeof({name}));')
        for member in members:
            lines.append(f'    printf("{member} %d\\n", (int){member});')
    lines += ["    return 0;", "}", ""]
    return "\n".join(lines)


def run(tmp_path, tag, source, flags):
    path, exe = tmp_path / f"{tag}.c", tmp_path / tag
    path.write_text(source)
    built = subprocess.run(["gcc", "-std=c11", "-w", *flags, str(path), "-o", str(exe)], capture_output=True,
                           text=True)
    assert built.returncode == 0, built.stderr[-3000:]
    return subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.splitlines()


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "include")) or not shutil.which("gcc"),
                    reason="needs the reference's headers and gcc")
def test_mirrored_types_have_the_reference_layout(tmp_path):
    structs, enums = parse_header()
    structs = {n: f for n, f in structs.items() if not OWN_TYPES.match(n)}
    enums = {n: [m for m in members if m not in ADDITIONS] for n, members in enums.items()
             if not OWN_TYPES.match(n)}
    assert len(structs) >= 20 and len(enums) >= 15
    ours = run(tmp_path, "ours", program(['"yvex_rocm.h"'], structs, enums),
               [f"-I{os.path.join(ROOT, 'include')}"])
    theirs = run(tmp_path, "theirs", program([f"<{h}>" for h in REFERENCE_HEADERS], structs, enums),
                 [f"-I{os.path.join(REFERENCE, 'include')}"])
    differing = [(a, b) for a, b in zip(ours, theirs) if a != b]
    assert not differing, differing[:20]
    assert len(ours) == len(theirs)


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "include")) or not shutil.which("gcc"),
                    reason="needs the reference's headers and gcc")
def test_renamed_types_have_the_reference_layout(tmp_path):
    """The operation facts and the MoE operations table carry the library's own names (their
    function pointers take its backend type) but the reference's members in the reference's order."""
    structs, _ = parse_header()
    ours = run(tmp_path, "ours", program(['"yvex_rocm.h"'], {n: structs[n] for n in RENAMED}, {}),
               [f"-I{os.path.join(ROOT, 'include')}"])
    theirs = run(tmp_path, "theirs", program([f"<{h}>" for h in REFERENCE_HEADERS],
                                             {RENAMED[n]: structs[n] for n in RENAMED}, {}),
                 [f"-I{os.path.join(REFERENCE, 'include')}"])
    for name, other in RENAMED.items():
        theirs = [line.replace(other, name) for line in theirs]
    assert ours == theirs and len(ours) > 20


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "src", "backend")) or not shutil.which("gcc"),
                    reason="needs the reference's sources and gcc")
def test_reference_side_adapter_compiles_against_the_reference():
    """The binding a maintainer adds to the reference tree: checked against the reference's own
    headers (the public ones and src/backend/private.h), with this library's header in the mode
    that takes the shared types from them. Warnings are errors."""
    built = subprocess.run(["gcc", "-std=c11", "-Wall", "-Wextra", "-Werror", "-fsyntax-only",
                            f"-I{os.path.join(REFERENCE, 'include')}", f"-I{os.path.join(REFERENCE, 'src')}",
                            f"-I{os.path.join(ROOT, 'include')}", ADAPTER], capture_output=True, text=True)
    assert built.returncode == 0, built.stderr[-3000:]
