module {
  func @tpu_func(%arg0: tensor<2x8x10x9xsi8>) -> tensor<2x24x10x9xsi8> {
    %0 = "tpu.weight_file"() {filename = "se_block_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.none"() : () -> none
    %2 = "tpu.input"(%arg0) {name = "input", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}} : (tensor<2x8x10x9xsi8>) -> tensor<2x8x10x9xsi8>
    %3 = "tpu.load_weight"(%0) {name = "c1_filter", storage = "INT8"} : (memref<10xf32>) -> tensor<24x8x3x3xf32>
    %4 = "tpu.load_weight"(%0) {name = "c1_bias", storage = "INT32"} : (memref<10xf32>) -> tensor<24xf32>
    %5 = "tpu.load_weight"(%0) {name = "c1_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<24xf32>
    %6 = "tpu.load_weight"(%0) {name = "c1_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<24xf32>
    %7 = "tpu.conv_2d"(%2, %3, %4, %1, %1, %5, %6) {name = "c1", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 0.000000e+00 : f32}, param = {dilation_h = 1 : i32, dilation_w = 1 : i32, group = 1 : i32, ins = [], is_dw = false, kernel_h = 3 : i32, kernel_w = 3 : i32, pad_value = 0 : i32, padding = "SAME", padding_b = 1 : i32, padding_l = 1 : i32, padding_r = 1 : i32, padding_t = 1 : i32, stride_h = 1 : i32, stride_w = 1 : i32, with_bias = true}, do_relu = true} : (tensor<2x8x10x9xsi8>, tensor<24x8x3x3xf32>, tensor<24xf32>, none, none, tensor<24xf32>, tensor<24xf32>) -> tensor<2x24x10x9xsi8>
    %8 = "tpu.load_weight"(%0) {name = "c2_filter", storage = "INT8"} : (memref<10xf32>) -> tensor<24x8x3x3xf32>
    %9 = "tpu.load_weight"(%0) {name = "c2_bias", storage = "INT32"} : (memref<10xf32>) -> tensor<24xf32>
    %10 = "tpu.load_weight"(%0) {name = "c2_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<24xf32>
    %11 = "tpu.load_weight"(%0) {name = "c2_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<24xf32>
    %12 = "tpu.conv_2d"(%2, %8, %9, %1, %1, %10, %11) {name = "c2", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 0.000000e+00 : f32}, param = {dilation_h = 1 : i32, dilation_w = 1 : i32, group = 1 : i32, ins = [], is_dw = false, kernel_h = 3 : i32, kernel_w = 3 : i32, pad_value = 0 : i32, padding = "SAME", padding_b = 1 : i32, padding_l = 1 : i32, padding_r = 1 : i32, padding_t = 1 : i32, stride_h = 1 : i32, stride_w = 1 : i32, with_bias = true}, do_relu = false} : (tensor<2x8x10x9xsi8>, tensor<24x8x3x3xf32>, tensor<24xf32>, none, none, tensor<24xf32>, tensor<24xf32>) -> tensor<2x24x10x9xsi8>
    %13 = "tpu.load_weight"(%0) {name = "pr_slope", storage = "INT8"} : (memref<10xf32>) -> tensor<24xf32>
    %14 = "tpu.load_weight"(%0) {name = "pr_rshift_pos", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %15 = "tpu.load_weight"(%0) {name = "pr_multiplier_pos", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %16 = "tpu.load_weight"(%0) {name = "pr_rshift_neg", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %17 = "tpu.prelu"(%12, %13, %1, %1, %1, %1, %14, %15, %16) {name = "pr", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 0.000000e+00 : f32}} : (tensor<2x24x10x9xsi8>, tensor<24xf32>, none, none, none, none, tensor<1xf32>, tensor<1xf32>, tensor<1xf32>) -> tensor<2x24x10x9xsi8>
    %18 = "tpu.load_weight"(%0) {name = "mx_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %19 = "tpu.load_weight"(%0) {name = "mx_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<2xf32>
    %20 = "tpu.eltwise_max"(%7, %12, %1, %1, %18, %19) {name = "mx", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 0.000000e+00 : f32}, do_relu = false} : (tensor<2x24x10x9xsi8>, tensor<2x24x10x9xsi8>, none, none, tensor<1xf32>, tensor<2xf32>) -> tensor<2x24x10x9xsi8>
    %21 = "tpu.load_weight"(%0) {name = "mn_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %22 = "tpu.load_weight"(%0) {name = "mn_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<2xf32>
    %23 = "tpu.eltwise_min"(%7, %17, %1, %1, %21, %22) {name = "mn", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 0.000000e+00 : f32}, do_relu = true} : (tensor<2x24x10x9xsi8>, tensor<2x24x10x9xsi8>, none, none, tensor<1xf32>, tensor<2xf32>) -> tensor<2x24x10x9xsi8>
    %24 = "tpu.load_weight"(%0) {name = "ml_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %25 = "tpu.load_weight"(%0) {name = "ml_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %26 = "tpu.eltwise_mul"(%20, %23, %1, %1, %24, %25) {name = "ml", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 0.000000e+00 : f32}, do_relu = false} : (tensor<2x24x10x9xsi8>, tensor<2x24x10x9xsi8>, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<2x24x10x9xsi8>
    %27 = "tpu.load_weight"(%0) {name = "gap_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %28 = "tpu.load_weight"(%0) {name = "gap_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %29 = "tpu.pool_avg_2d"(%26, %1, %1, %27, %28) {name = "gap", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 0.000000e+00 : f32}, param = {count_include_pad = true, kernel_h = 10 : i32, kernel_w = 9 : i32, pad_value = 0 : i32, padding_b = 0 : i32, padding_l = 0 : i32, padding_r = 0 : i32, padding_t = 0 : i32, stride_h = 1 : i32, stride_w = 1 : i32}, do_relu = false} : (tensor<2x24x10x9xsi8>, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<2x24x1x1xsi8>
    %30 = "tpu.load_weight"(%0) {name = "gate_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %31 = "tpu.load_weight"(%0) {name = "gate_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %32 = "tpu.broadcast_mul"(%20, %29, %1, %1, %30, %31) {name = "gate", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 0.000000e+00 : f32}, do_relu = false} : (tensor<2x24x10x9xsi8>, tensor<2x24x1x1xsi8>, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<2x24x10x9xsi8>
    %33 = "tpu.load_weight"(%0) {name = "badd_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %34 = "tpu.load_weight"(%0) {name = "badd_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<2xf32>
    %35 = "tpu.broadcast_add"(%32, %29, %1, %1, %33, %34) {name = "badd", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 0.000000e+00 : f32}, do_relu = true} : (tensor<2x24x10x9xsi8>, tensor<2x24x1x1xsi8>, none, none, tensor<1xf32>, tensor<2xf32>) -> tensor<2x24x10x9xsi8>
    %36 = "tpu.load_weight"(%0) {name = "bsub_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %37 = "tpu.load_weight"(%0) {name = "bsub_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<2xf32>
    %38 = "tpu.broadcast_sub"(%29, %35, %1, %1, %36, %37) {name = "bsub", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 0.000000e+00 : f32}, do_relu = false} : (tensor<2x24x1x1xsi8>, tensor<2x24x10x9xsi8>, none, none, tensor<1xf32>, tensor<2xf32>) -> tensor<2x24x10x9xsi8>
    %39 = "tpu.load_weight"(%0) {name = "sig_table", storage = "INT8"} : (memref<10xf32>) -> tensor<256xf32>
    %40 = "tpu.sigmoid"(%38, %39, %1) {name = "sig", quant = {mode = "INT8", param_type = "LUT_INT8", threshold = 0.000000e+00 : f32}} : (tensor<2x24x10x9xsi8>, tensor<256xf32>, none) -> tensor<2x24x10x9xsi8>
    return %40 : tensor<2x24x10x9xsi8>
  }
}
