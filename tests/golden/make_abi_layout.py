"""Writes abi_layout.json: sizes and field offsets of the structs that Ocean's interface layer and
its GPU device module share, taken from the REFERENCE's own headers (compiled in this container,
where /root/reference is mounted). The field list is host/abi_layout_fields.h; the unary and
binary table entries come from the reference's generate_tensor_{unary,binary}.h, so the order of
the function table is the reference's, not ours.

    python tests/golden/make_abi_layout.py
"""
import json
import os
import subprocess
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REF = "/root/reference/include"
HOST = os.path.join(ROOT, "ocean-tensor-package_amd", "host")

PROBE = r'''
#include "ocean/core/interface/module_core.h"
#include <stdio.h>
#include <stddef.h>
#define OC_UNARY_TABLE(X)  UNARY_FROM_REFERENCE
#define OC_BINARY_TABLE(X) BINARY_FROM_REFERENCE
#define OC_AXIS_TABLE(X) X(axisAny,0) X(axisAll,0) X(axisAllFinite,0) X(axisAnyInf,0) X(axisAnyNaN,0) X(axisNnz,0) X(axisNnzNaN,0) \
   X(axisSum,0) X(axisProd,0) X(axisSumNaN,0) X(axisProdNaN,0) X(axisSumAbs,0) X(axisSumAbsNaN,0) X(axisMinimum,0) X(axisMaximum,0) \
   X(axisMinimumAbs,0) X(axisMaximumAbs,0) X(axisNorm2,0) X(axisNorm2NaN,0)
int main(void)
{  int first = 1;
   printf("{");
#define S(T)    printf("%s\"sizeof(" #T ")\": %zu", first ? "" : ", ", sizeof(T)); first = 0;
#define F(T, M) printf(", \"" #T "." #M "\": %zu", offsetof(T, M));
#include "abi_layout_fields.h"
   printf("}\n");
   return 0;
}
'''


def names(header):
    out = []
    for line in open(os.path.join(REF, "ocean/core/generic", header)):
        line = line.strip()
        if line.startswith("OC_TEMPLATE("):
            out.append(line[len("OC_TEMPLATE("):].split(",")[0].strip())
    return out


def main():
    unary = " ".join("X(%s,0)" % n for n in names("generate_tensor_unary.h"))
    binary = " ".join("X(%s,0)" % n for n in names("generate_tensor_binary.h"))
    src = PROBE.replace("UNARY_FROM_REFERENCE", unary).replace("BINARY_FROM_REFERENCE", binary)
    with tempfile.TemporaryDirectory() as tmp:
        c = os.path.join(tmp, "probe.c")
        open(c, "w").write(src)
        exe = os.path.join(tmp, "probe")
        subprocess.run(["gcc", "-I" + REF, "-I" + HOST, c, "-o", exe], check=True)
        layout = json.loads(subprocess.run([exe], check=True, capture_output=True, text=True).stdout)
    layout["_unary_order"] = names("generate_tensor_unary.h")
    layout["_binary_order"] = names("generate_tensor_binary.h")
    with open(os.path.join(HERE, "abi_layout.json"), "w") as f:
        json.dump(layout, f, indent=0, sort_keys=True)
    print("wrote abi_layout.json with %d entries" % len(layout))


if __name__ == "__main__":
    main()
