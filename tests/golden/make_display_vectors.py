"""Writes tests/golden/display_vectors.json: the expected-output string literals of the reference's
display tests (tests/tensor/test_display.nim) for integer and float tensors, each with a description of
the input that produces it. Data only: inputs as (generator, arguments), outputs as the literal text.
Runs where the reference tree is present (/root/reference); the JSON it writes is what the tests read.

    python tests/golden/make_display_vectors.py
"""
import json
import os
import re

REF = "/root/reference/tests/tensor/test_display.nim"
HERE = os.path.dirname(os.path.abspath(__file__))

# (test name in the reference file, ordinal of the `compareStrings(` / `check` literal inside it, input, call)
CASES = [
    ("Display 1D tensor", 0, dict(values=[0.9532932, 0.12945823], dtype="f64", shape=[2]), dict(specifier="")),
    ("Display 1D tensor", 1, dict(values=[0.9532932, 0.12945823], dtype="f64", shape=[2]), dict(specifier="<:>")),
    ("Display 1D tensor", 2, dict(values=[1, 2, 3, 4], dtype="i64", shape=[4]), dict(specifier="")),
    ("Display 1D tensor", 3, dict(values=[1, 2, 3, 4], dtype="i64", shape=[4]), dict(specifier="<:>")),
    ("Display 2D tensor (single-column)", 0, dict(arange=[1, 6], dtype="i64", shape=[1, 5]), dict(specifier="")),
    ("Display 2D tensor (single-column)", 1, dict(arange=[1, 6], dtype="i64", shape=[1, 5]), dict(specifier="<:>")),
    ("Display 2D tensor (single-column)", 2, dict(arange=[1, 6], dtype="i64", shape=[5, 1]), dict(specifier="")),
    ("Display 2D tensor (single-column)", 3, dict(arange=[1, 6], dtype="i64", shape=[5, 1]), dict(specifier="<:>")),
    ("Display 2D tensor (multi-column)", 0, dict(vandermonde=5, dtype="i64", shape=[5, 5]), dict(specifier="")),
    ("Display 2D tensor (multi-column)", 1, dict(vandermonde=5, dtype="i64", shape=[5, 5]), dict(specifier="<:>")),
    ("Display 3D tensor", 0, dict(arange=[1, 25], dtype="i64", shape=[2, 3, 4]), dict(specifier="")),
    ("Display 3D tensor", 1, dict(arange=[1, 25], dtype="i64", shape=[2, 3, 4]), dict(specifier="<:>")),
    ("Display 4D tensor", 0, dict(arange=[1, 73], dtype="i64", shape=[2, 3, 4, 3]), dict(specifier="")),
    ("Display 4D tensor", 1, dict(arange=[1, 73], dtype="i64", shape=[2, 3, 4, 3]), dict(specifier="<:>")),
    ("Display 4D tensor with float values", 0, dict(linspace=[0.0, 100.0, 72], dtype="f64", shape=[2, 3, 4, 3]), dict(specifier="")),
    ("Display 4D tensor with float values", 1, dict(linspace=[0.0, 100.0, 72], dtype="f64", shape=[2, 3, 4, 3]), dict(specifier="<:>")),
    ("Display 4D tensor with float values and custom precision", 0, dict(linspace=[0.0, 100.0, 72], dtype="f64", shape=[2, 3, 4, 3]),
     dict(specifier="", precision=4)),
    ("Display 5D tensor", 0, dict(arange=[1, 145], dtype="i64", shape=[2, 3, 4, 3, 2]), dict(specifier="")),
    ("Display 5D tensor", 1, dict(arange=[1, 145], dtype="i64", shape=[2, 2, 1, 3, 12]), dict(specifier="<:>")),
    ("Display 5D tensor", 2, dict(arange=[1, 217], dtype="i64", shape=[3, 3, 4, 3, 2]), dict(specifier="")),
    ("Display 5D tensor with large numbers", 0, dict(arange=[1000000000, 1000000216], dtype="i64", shape=[3, 3, 4, 3, 2]), dict(specifier="")),
    ("Display 5D tensor with large numbers", 1, dict(arange=[1000000000, 1000000216], dtype="i64", shape=[2, 3, 1, 6, 6]), dict(specifier="<:>")),
    ("Format-strings (3D tensor)", 0, dict(arange=[-2, 10], dtype="i64", shape=[2, 2, 3]), dict(specifier="")),
    ("Format-strings (3D tensor)", 1, dict(arange=[-2, 10], dtype="i64", shape=[2, 2, 3]), dict(specifier="||")),
    ("Format-strings (3D tensor)", 2, dict(arange=[-2, 10], dtype="i64", shape=[2, 2, 3]), dict(specifier="[:]")),
    ("Format-strings (3D tensor)", 3, dict(arange=[-2, 10], dtype="i64", shape=[2, 2, 3]), dict(specifier="<:>")),
]
# single-line `check &"{t:...}" == "..."` literals of the two format-string tests
EXACT = [
    ("Format-strings (1D tensor)", dict(arange=[-2, 10], dtype="i64", shape=[12]), [
        ("||", "    -2    -1     0     1     2     3     4     5     6     7     8     9"),
        ("[]", "[-2, -1, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9]"),
        ("<>", "Tensor[int]<12>:[-2, -1, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9]"),
        ("[:]", "[-2, -1, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9]"),
        ("<:>", "Tensor[int]<12>:\n[-2, -1, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9]")]),
    ("Format-strings (3D tensor)", dict(arange=[-2, 10], dtype="i64", shape=[2, 2, 3]), [
        ("[]", "[[[-2, -1, 0], [1, 2, 3]], [[4, 5, 6], [7, 8, 9]]]"),
        ("<>", "Tensor[int]<2,2,3>:[[[-2, -1, 0], [1, 2, 3]], [[4, 5, 6], [7, 8, 9]]]")]),
]


def main():
    text = open(REF).read()
    tests = {}
    for m in re.finditer(r'    test "([^"]+)":\n(.*?)(?=\n    test "|\nmain\(\))', text, flags=re.S):
        tests[m.group(1)] = re.findall(r'compareStrings\([^\n]*?, """(.*?)"""\)', m.group(2), flags=re.S)
    out = {"_about": "Expected-output literals of the reference's tests/tensor/test_display.nim (the reference compares line "
                     "by line after stripping each line, `compareStrings`, :18-23); `exact` cases are compared with ==. The "
                     "header of a device tensor names its own type and backend in place of Tensor / Cpu.",
           "compare_strings": [], "exact": []}
    for name, k, inp, call in CASES:
        lit = tests[name][k]
        for spec_check in EXACT:
            assert all(e[1] in text.replace("\\n", "\n") for e in spec_check[2]), spec_check[0]
        out["compare_strings"].append(dict(source=f"test_display.nim, test \"{name}\", literal {k}", input=inp, call=call, expect=lit))
    for name, inp, pairs in EXACT:
        for spec, lit in pairs:
            out["exact"].append(dict(source=f"test_display.nim, test \"{name}\"", input=inp, call=dict(specifier=spec), expect=lit))
    with open(os.path.join(HERE, "display_vectors.json"), "w") as f:
        json.dump(out, f, indent=1)
    print(len(out["compare_strings"]), "compareStrings literals,", len(out["exact"]), "exact literals")


if __name__ == "__main__":
    main()
