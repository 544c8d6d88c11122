"""Writes tests/golden/resnet18_reduce_ops.mlir: every `byre.compute @Reduce*` line of the
reference's three ResNet-18 host modules (runtime/test/test_files/resnet18_{fw_bw,fw,bw}_host_cuda.mlir),
copied character for character, inside one entry function whose arguments are the ops' operands.
The lines are data produced by the reference's compiler: attribute spelling (`dense<[3, 2]>`,
`memory_effects`), operand types (rank-0 results, f16) and op keys are what a real module
carries.  Run here, where the reference checkout is mounted; the output is committed."""
import os
import re
import sys

SRC = "/root/reference/runtime/test/test_files"
FILES = ["resnet18_fw_bw_host_cuda.mlir", "resnet18_fw_host_cuda.mlir", "resnet18_bw_host_cuda.mlir"]


def main():
    ops = []
    for f in FILES:
        for n, line in enumerate(open(os.path.join(SRC, f)), 1):
            if "byre.compute @Reduce" in line:
                ops.append((f, n, line.rstrip("\n")))
    args, body = [], []
    for i, (f, n, line) in enumerate(ops):
        m = re.match(r"(\s*byre\.compute @\w+)\((%\w+), (%\w+)\)( \{.*\} : )(memref<[^>]*>), (memref<[^>]*>)\s*$", line)
        assert m, line
        head, _, _, attrs, t_in, t_out = m.groups()
        a_in, a_out = f"%arg{2 * i}", f"%arg{2 * i + 1}"
        args.append(f'{a_in}: {t_in} {{byre.argname = "In{i}", byre.argtype = 1 : i32}}')
        args.append(f'{a_out}: {t_out} {{byre.argname = "Out{i}", byre.argtype = 2 : i32}}')
        # only the two SSA names change; key, attributes and types stay as the compiler wrote them
        body.append(f"    // {f}:{n}")
        body.append(f"{head}({a_in}, {a_out}){attrs}{t_in}, {t_out}")
    out = ["module attributes {byre.container_module} {",
           "  func.func @main(" + ", ".join(args) + ") attributes {byre.entry_point} {",
           *body, "    return", "  }", "}", ""]
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "resnet18_reduce_ops.mlir")
    open(path, "w").write("\n".join(out))
    print(f"{len(ops)} ops -> {path}")


if __name__ == "__main__":
    sys.exit(main())
