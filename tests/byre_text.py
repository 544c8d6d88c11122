"""Builds ByRE module text for one-op tests, the job the reference's in-memory ByREBuilder does
for its op tests (runtime/test/common/models.cc:893-931 for reductions)."""


def memref(shape, dtype, space):
    dims = "x".join(str(d) for d in shape)
    return f'memref<{dims + "x" if shape else ""}{dtype}, "{space}">'


def reduction_module(space, shape, dims, op_name, dtype="f32", dense=True):
    out_shape = [s for i, s in enumerate(shape) if i not in dims]
    tin, tout = memref(shape, dtype, space), memref(out_shape, dtype, space)
    if dense:
        attr = f"dense<[{', '.join(str(d) for d in dims)}]> : tensor<{len(dims)}xi64>"
    else:
        attr = "[" + ", ".join(f"{d} : i64" for d in dims) + "]"
    return f"""module attributes {{byre.container_module}} {{
  func.func @test(%arg0 : {tin} {{byre.argname = "A", byre.argtype = 1: i32}},
                  %arg1 : {tout} {{byre.argname = "B", byre.argtype = 2: i32}}) attributes {{byre.entry_point}} {{
    byre.compute @{op_name}(%arg0, %arg1) {{dimensions = {attr}, memory_effects = [1 : i32, 2 : i32]}} : {tin}, {tout}
    return
  }}
}}
"""


def softmax_module(space, shape, dtype, axis):
    t = memref(shape, dtype, space)
    return f"""module attributes {{byre.container_module}} {{
  func.func @test(%arg0 : {t} {{byre.argname = "X", byre.argtype = 1: i32}},
                  %arg1 : {t} {{byre.argname = "Y", byre.argtype = 2: i32}}) attributes {{byre.entry_point}} {{
    byre.compute @byteir.softmax(%arg0, %arg1) {{axis = {axis} : i64, device = "cuda"}} : {t}, {t}
    return
  }}
}}
"""
