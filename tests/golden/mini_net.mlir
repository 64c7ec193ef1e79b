module {
  func @tpu_func(%arg0: tensor<2x3x40x40xsi8>) -> tensor<2x10xsi8> {
    %0 = "tpu.weight_file"() {filename = "mini_net_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.none"() : () -> none
    %2 = "tpu.input"(%arg0) {name = "input", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}} : (tensor<2x3x40x40xsi8>) -> tensor<2x3x40x40xsi8>
    %3 = "tpu.load_weight"(%0) {name = "stem_filter", storage = "INT8"} : (memref<10xf32>) -> tensor<16x3x3x3xf32>
    %4 = "tpu.load_weight"(%0) {name = "stem_bias", storage = "INT32"} : (memref<10xf32>) -> tensor<16xf32>
    %5 = "tpu.load_weight"(%0) {name = "stem_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<16xf32>
    %6 = "tpu.load_weight"(%0) {name = "stem_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<16xf32>
    %7 = "tpu.conv_2d"(%2, %3, %4, %1, %1, %5, %6) {name = "stem", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 0.000000e+00 : f32}, param = {dilation_h = 1 : i32, dilation_w = 1 : i32, group = 1 : i32, ins = [], is_dw = false, kernel_h = 3 : i32, kernel_w = 3 : i32, pad_value = 0 : i32, padding = "SAME", padding_b = 1 : i32, padding_l = 1 : i32, padding_r = 1 : i32, padding_t = 1 : i32, stride_h = 2 : i32, stride_w = 2 : i32, with_bias = true}, do_relu = false} : (tensor<2x3x40x40xsi8>, tensor<16x3x3x3xf32>, tensor<16xf32>, none, none, tensor<16xf32>, tensor<16xf32>) -> tensor<2x16x20x20xsi8>
    %8 = "tpu.load_weight"(%0) {name = "stem_leaky_rshift_pos", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %9 = "tpu.load_weight"(%0) {name = "stem_leaky_multiplier_pos", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %10 = "tpu.load_weight"(%0) {name = "stem_leaky_rshift_neg", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %11 = "tpu.load_weight"(%0) {name = "stem_leaky_multiplier_neg", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %12 = "tpu.leaky_relu"(%7, %1, %1, %1, %1, %8, %9, %10, %11) {name = "stem_leaky", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 0.000000e+00 : f32}, negative_slope = 1.000000e-01 : f32} : (tensor<2x16x20x20xsi8>, none, none, none, none, tensor<1xf32>, tensor<1xf32>, tensor<1xf32>, tensor<1xf32>) -> tensor<2x16x20x20xsi8>
    %13 = "tpu.pool_max_2d"(%12) {name = "pool", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}, param = {count_include_pad = false, kernel_h = 3 : i32, kernel_w = 3 : i32, pad_value = 0 : i32, padding_b = 1 : i32, padding_l = 0 : i32, padding_r = 1 : i32, padding_t = 0 : i32, stride_h = 2 : i32, stride_w = 2 : i32}, do_relu = false} : (tensor<2x16x20x20xsi8>) -> tensor<2x16x10x10xsi8>
    %14 = "tpu.load_weight"(%0) {name = "expand_filter", storage = "INT8"} : (memref<10xf32>) -> tensor<48x16x1x1xf32>
    %15 = "tpu.load_weight"(%0) {name = "expand_bias", storage = "INT32"} : (memref<10xf32>) -> tensor<48xf32>
    %16 = "tpu.load_weight"(%0) {name = "expand_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<48xf32>
    %17 = "tpu.load_weight"(%0) {name = "expand_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<48xf32>
    %18 = "tpu.conv_2d"(%13, %14, %15, %1, %1, %16, %17) {name = "expand", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 0.000000e+00 : f32}, param = {dilation_h = 1 : i32, dilation_w = 1 : i32, group = 1 : i32, ins = [], is_dw = false, kernel_h = 1 : i32, kernel_w = 1 : i32, pad_value = 0 : i32, padding = "SAME", padding_b = 0 : i32, padding_l = 0 : i32, padding_r = 0 : i32, padding_t = 0 : i32, stride_h = 1 : i32, stride_w = 1 : i32, with_bias = true}, do_relu = true} : (tensor<2x16x10x10xsi8>, tensor<48x16x1x1xf32>, tensor<48xf32>, none, none, tensor<48xf32>, tensor<48xf32>) -> tensor<2x48x10x10xsi8>
    %19 = "tpu.load_weight"(%0) {name = "dw_filter", storage = "INT8"} : (memref<10xf32>) -> tensor<48x1x1x3x3xf32>
    %20 = "tpu.load_weight"(%0) {name = "dw_bias", storage = "INT32"} : (memref<10xf32>) -> tensor<48xf32>
    %21 = "tpu.load_weight"(%0) {name = "dw_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<48xf32>
    %22 = "tpu.load_weight"(%0) {name = "dw_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<48xf32>
    %23 = "tpu.conv_2d"(%18, %19, %20, %1, %1, %21, %22) {name = "dw", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 0.000000e+00 : f32}, param = {dilation_h = 1 : i32, dilation_w = 1 : i32, group = 48 : i32, ins = [], is_dw = true, kernel_h = 3 : i32, kernel_w = 3 : i32, pad_value = 0 : i32, padding = "SAME", padding_b = 1 : i32, padding_l = 1 : i32, padding_r = 1 : i32, padding_t = 1 : i32, stride_h = 1 : i32, stride_w = 1 : i32, with_bias = true}, do_relu = true} : (tensor<2x48x10x10xsi8>, tensor<48x1x1x3x3xf32>, tensor<48xf32>, none, none, tensor<48xf32>, tensor<48xf32>) -> tensor<2x48x10x10xsi8>
    %24 = "tpu.load_weight"(%0) {name = "project_filter", storage = "INT8"} : (memref<10xf32>) -> tensor<16x48x1x1xf32>
    %25 = "tpu.load_weight"(%0) {name = "project_bias", storage = "INT32"} : (memref<10xf32>) -> tensor<16xf32>
    %26 = "tpu.load_weight"(%0) {name = "project_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<16xf32>
    %27 = "tpu.load_weight"(%0) {name = "project_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<16xf32>
    %28 = "tpu.conv_2d"(%23, %24, %25, %1, %1, %26, %27) {name = "project", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 0.000000e+00 : f32}, param = {dilation_h = 1 : i32, dilation_w = 1 : i32, group = 1 : i32, ins = [], is_dw = false, kernel_h = 1 : i32, kernel_w = 1 : i32, pad_value = 0 : i32, padding = "SAME", padding_b = 0 : i32, padding_l = 0 : i32, padding_r = 0 : i32, padding_t = 0 : i32, stride_h = 1 : i32, stride_w = 1 : i32, with_bias = true}, do_relu = false} : (tensor<2x48x10x10xsi8>, tensor<16x48x1x1xf32>, tensor<16xf32>, none, none, tensor<16xf32>, tensor<16xf32>) -> tensor<2x16x10x10xsi8>
    %29 = "tpu.load_weight"(%0) {name = "res_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %30 = "tpu.load_weight"(%0) {name = "res_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<2xf32>
    %31 = "tpu.eltwise_add"(%28, %13, %1, %1, %29, %30) {name = "res", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 0.000000e+00 : f32}, do_relu = true} : (tensor<2x16x10x10xsi8>, tensor<2x16x10x10xsi8>, none, none, tensor<1xf32>, tensor<2xf32>) -> tensor<2x16x10x10xsi8>
    %32 = "tpu.load_weight"(%0) {name = "down_filter", storage = "INT8"} : (memref<10xf32>) -> tensor<32x16x3x3xf32>
    %33 = "tpu.load_weight"(%0) {name = "down_bias", storage = "INT32"} : (memref<10xf32>) -> tensor<32xf32>
    %34 = "tpu.load_weight"(%0) {name = "down_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<32xf32>
    %35 = "tpu.load_weight"(%0) {name = "down_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<32xf32>
    %36 = "tpu.conv_2d"(%31, %32, %33, %1, %1, %34, %35) {name = "down", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 0.000000e+00 : f32}, param = {dilation_h = 1 : i32, dilation_w = 1 : i32, group = 1 : i32, ins = [], is_dw = false, kernel_h = 3 : i32, kernel_w = 3 : i32, pad_value = 0 : i32, padding = "SAME", padding_b = 0 : i32, padding_l = 1 : i32, padding_r = 0 : i32, padding_t = 1 : i32, stride_h = 2 : i32, stride_w = 2 : i32, with_bias = true}, do_relu = true} : (tensor<2x16x10x10xsi8>, tensor<32x16x3x3xf32>, tensor<32xf32>, none, none, tensor<32xf32>, tensor<32xf32>) -> tensor<2x32x5x5xsi8>
    %37 = "tpu.upsample"(%36) {name = "up", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}, scale_h = 2 : i32, scale_w = 2 : i32} : (tensor<2x32x5x5xsi8>) -> tensor<2x32x10x10xsi8>
    %38 = "tpu.concat"(%37, %31, %1, %1, %1, %1) {name = "cat", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}, axis = 1 : i32, do_relu = false} : (tensor<2x32x10x10xsi8>, tensor<2x16x10x10xsi8>, none, none, none, none) -> tensor<2x48x10x10xsi8>
    %39 = "tpu.load_weight"(%0) {name = "head_filter", storage = "INT8"} : (memref<10xf32>) -> tensor<40x48x1x3xf32>
    %40 = "tpu.load_weight"(%0) {name = "head_bias", storage = "INT32"} : (memref<10xf32>) -> tensor<40xf32>
    %41 = "tpu.load_weight"(%0) {name = "head_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<40xf32>
    %42 = "tpu.load_weight"(%0) {name = "head_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<40xf32>
    %43 = "tpu.conv_2d"(%38, %39, %40, %1, %1, %41, %42) {name = "head", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 0.000000e+00 : f32}, param = {dilation_h = 1 : i32, dilation_w = 1 : i32, group = 1 : i32, ins = [], is_dw = false, kernel_h = 1 : i32, kernel_w = 3 : i32, pad_value = 0 : i32, padding = "SAME", padding_b = 0 : i32, padding_l = 1 : i32, padding_r = 1 : i32, padding_t = 0 : i32, stride_h = 1 : i32, stride_w = 1 : i32, with_bias = true}, do_relu = true} : (tensor<2x48x10x10xsi8>, tensor<40x48x1x3xf32>, tensor<40xf32>, none, none, tensor<40xf32>, tensor<40xf32>) -> tensor<2x40x10x10xsi8>
    %44 = "tpu.load_weight"(%0) {name = "head_clip_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %45 = "tpu.load_weight"(%0) {name = "head_clip_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %46 = "tpu.clip"(%43, %1, %1, %44, %45) {name = "head_clip", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 0.000000e+00 : f32}, max = 9.000000e+01 : f32, min = 0.000000e+00 : f32} : (tensor<2x40x10x10xsi8>, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<2x40x10x10xsi8>
    %47 = "tpu.load_weight"(%0) {name = "gap_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %48 = "tpu.load_weight"(%0) {name = "gap_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %49 = "tpu.pool_avg_2d"(%46, %1, %1, %47, %48) {name = "gap", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 0.000000e+00 : f32}, param = {count_include_pad = true, kernel_h = 10 : i32, kernel_w = 10 : i32, pad_value = 0 : i32, padding_b = 0 : i32, padding_l = 0 : i32, padding_r = 0 : i32, padding_t = 0 : i32, stride_h = 1 : i32, stride_w = 1 : i32}, do_relu = false} : (tensor<2x40x10x10xsi8>, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<2x40x1x1xsi8>
    %50 = "tpu.reshape"(%49) {name = "flat", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}} : (tensor<2x40x1x1xsi8>) -> tensor<2x40xsi8>
    %51 = "tpu.load_weight"(%0) {name = "fc_filter", storage = "INT8"} : (memref<10xf32>) -> tensor<10x40xf32>
    %52 = "tpu.load_weight"(%0) {name = "fc_bias", storage = "INT32"} : (memref<10xf32>) -> tensor<10xf32>
    %53 = "tpu.load_weight"(%0) {name = "fc_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %54 = "tpu.load_weight"(%0) {name = "fc_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %55 = "tpu.fully_connected"(%50, %51, %52, %1, %1, %53, %54) {name = "fc", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 0.000000e+00 : f32}, do_relu = false} : (tensor<2x40xsi8>, tensor<10x40xf32>, tensor<10xf32>, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<2x10xsi8>
    return %55 : tensor<2x10xsi8>
  }
}
