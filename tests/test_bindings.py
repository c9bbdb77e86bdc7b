"""The Python binding declares the argument types of every C entry point; this checks the
declarations against the prototypes in the HIP sources, so that a changed kernel signature
cannot reach the GPU with arguments in the wrong places (no GPU needed)."""

from __future__ import annotations

import re
from pathlib import Path

from llmserve_amd.kernels.build import CSRC, FLAGS, library_name
from llmserve_amd.kernels.hip import _SIGNATURES
from llmserve_amd.kernels.variants import DEFAULT_VARIANTS


def prototypes() -> dict[str, str]:
    text = "\n".join(path.read_text() for path in sorted(CSRC.glob("*.hip")))
    found = {}
    for match in re.finditer(r'extern "C" int (\w+)\((.*?)\)\s*\{', text, re.S):
        arguments = [a.strip() for a in match.group(2).replace("\n", " ").split(",") if a.strip()]
        codes = ""
        for argument in arguments:
            if "*" in argument or "hipStream_t" in argument:
                codes += "p"
            elif argument.startswith("float"):
                codes += "f"
            elif argument.startswith("int"):
                codes += "i"
            else:
                codes += "?"
        found[match.group(1)] = codes
    return found


def test_declared_signatures_are_the_prototypes():
    found = prototypes()
    for name, signature in _SIGNATURES.items():
        assert found.get(name) == signature, name
    launched = {name for name, codes in found.items() if codes.endswith("p") and len(codes) > 1}
    assert launched <= set(_SIGNATURES), launched - set(_SIGNATURES)  # every launcher is declared


def test_build_names_depend_on_source_flags_and_constants():
    assert "--offload-arch=gfx950" in FLAGS and "-packed-fp32-ops" in FLAGS
    a = library_name("attention_bf16", {"HEAD_DIM": 64})
    b = library_name("attention_bf16", {"HEAD_DIM": 128})
    assert a != b and a.startswith("attention_bf16-head_dim64-") and a.endswith(".so")
    assert library_name("elementwise") == library_name("elementwise", {})
    for module in DEFAULT_VARIANTS:
        assert (CSRC / f"{module}.hip").is_file()
    assert Path(CSRC / "common.h").is_file()
