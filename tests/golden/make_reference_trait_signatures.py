"""Writes tests/golden/reference_trait_signatures.json: every method signature of the reference's `trait Backend` and
`trait BackendMatMul` (libs/rtensors/src/backend/mod.rs:216-485), with `specify_trait_unary_cabal!` / `specify_trait_scalar_cabal!`
expanded, reduced to tokens (name, generics, argument names and types, return type, where clause, whether the trait gives a default
body).  The reference's source is read as text here, in the container that holds it; tests read only the JSON.

    python tests/golden/make_reference_trait_signatures.py [/root/reference]
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import rust_sig  # noqa: E402


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    src = os.path.join(ref, "libs", "rtensors", "src", "backend", "mod.rs")
    text = rust_sig.expand(rust_sig.strip_comments(open(src).read()))
    out = {
        "source": "libs/rtensors/src/backend/mod.rs:216-485",
        "Backend": rust_sig.functions(rust_sig.block_of(text, r"pub\s+trait\s+Backend\s*:[^{]*\{")),
        "BackendMatMul": rust_sig.functions(rust_sig.block_of(text, r"pub\s+trait\s+BackendMatMul\s*<[^{]*\{")),
    }
    with open(os.path.join(HERE, "reference_trait_signatures.json"), "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    print(len(out["Backend"]), "methods of Backend,", len(out["BackendMatMul"]), "of BackendMatMul")


if __name__ == "__main__":
    main()
