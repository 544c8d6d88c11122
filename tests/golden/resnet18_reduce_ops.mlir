module attributes {byre.container_module} {
  func.func @main(%arg0: memref<4x1000xf16, "cuda"> {byre.argname = "In0", byre.argtype = 1 : i32}, %arg1: memref<4xf16, "cuda"> {byre.argname = "Out0", byre.argtype = 2 : i32}, %arg2: memref<4x512x7x7xf16, "cuda"> {byre.argname = "In1", byre.argtype = 1 : i32}, %arg3: memref<4x512xf16, "cuda"> {byre.argname = "Out1", byre.argtype = 2 : i32}, %arg4: memref<4x1000xf16, "cuda"> {byre.argname = "In2", byre.argtype = 1 : i32}, %arg5: memref<4xf16, "cuda"> {byre.argname = "Out2", byre.argtype = 2 : i32}, %arg6: memref<4x1000xf16, "cuda"> {byre.argname = "In3", byre.argtype = 1 : i32}, %arg7: memref<4xf16, "cuda"> {byre.argname = "Out3", byre.argtype = 2 : i32}, %arg8: memref<4x1000xf32, "cuda"> {byre.argname = "In4", byre.argtype = 1 : i32}, %arg9: memref<f32, "cuda"> {byre.argname = "Out4", byre.argtype = 2 : i32}, %arg10: memref<4x1000xf32, "cuda"> {byre.argname = "In5", byre.argtype = 1 : i32}, %arg11: memref<1000xf32, "cuda"> {byre.argname = "Out5", byre.argtype = 2 : i32}, %arg12: memref<1x512x7x7xf16, "cuda"> {byre.argname = "In6", byre.argtype = 1 : i32}, %arg13: memref<1x512xf16, "cuda"> {byre.argname = "Out6", byre.argtype = 2 : i32}, %arg14: memref<1x1000xf32, "cuda"> {byre.argname = "In7", byre.argtype = 1 : i32}, %arg15: memref<1000xf32, "cuda"> {byre.argname = "Out7", byre.argtype = 2 : i32}) attributes {byre.entry_point} {
    // resnet18_fw_bw_host_cuda.mlir:59
    byre.compute @ReduceSumOp_f16_f16(%arg0, %arg1) {device = "cuda", dimensions = dense<1> : tensor<1xi64>, memory_effects = [1 : i32, 2 : i32]} : memref<4x1000xf16, "cuda">, memref<4xf16, "cuda">
    // resnet18_fw_bw_host_cuda.mlir:178
    byre.compute @ReduceSumOp_f16_f16(%arg2, %arg3) {device = "cuda", dimensions = dense<[3, 2]> : tensor<2xi64>, memory_effects = [1 : i32, 2 : i32]} : memref<4x512x7x7xf16, "cuda">, memref<4x512xf16, "cuda">
    // resnet18_fw_bw_host_cuda.mlir:186
    byre.compute @ReduceMaxOp_f16_f16(%arg4, %arg5) {device = "cuda", dimensions = dense<1> : tensor<1xi64>, memory_effects = [1 : i32, 2 : i32]} : memref<4x1000xf16, "cuda">, memref<4xf16, "cuda">
    // resnet18_fw_bw_host_cuda.mlir:190
    byre.compute @ReduceSumOp_f16_f16(%arg6, %arg7) {device = "cuda", dimensions = dense<1> : tensor<1xi64>, memory_effects = [1 : i32, 2 : i32]} : memref<4x1000xf16, "cuda">, memref<4xf16, "cuda">
    // resnet18_fw_bw_host_cuda.mlir:300
    byre.compute @ReduceSumOp_f32_f32(%arg8, %arg9) {device = "cuda", dimensions = dense<[0, 1]> : tensor<2xi64>, memory_effects = [1 : i32, 2 : i32]} : memref<4x1000xf32, "cuda">, memref<f32, "cuda">
    // resnet18_fw_bw_host_cuda.mlir:326
    byre.compute @ReduceSumOp_f32_f32(%arg10, %arg11) {device = "cuda", dimensions = dense<0> : tensor<1xi64>, memory_effects = [1 : i32, 2 : i32]} : memref<4x1000xf32, "cuda">, memref<1000xf32, "cuda">
    // resnet18_fw_host_cuda.mlir:136
    byre.compute @ReduceSumOp_f16_f16(%arg12, %arg13) {device = "cuda", dimensions = dense<[3, 2]> : tensor<2xi64>, memory_effects = [1 : i32, 2 : i32]} : memref<1x512x7x7xf16, "cuda">, memref<1x512xf16, "cuda">
    // resnet18_bw_host_cuda.mlir:138
    byre.compute @ReduceSumOp_f32_f32(%arg14, %arg15) {device = "cuda", dimensions = dense<0> : tensor<1xi64>, memory_effects = [1 : i32, 2 : i32]} : memref<1x1000xf32, "cuda">, memref<1000xf32, "cuda">
    return
  }
}
