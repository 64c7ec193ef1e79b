module {
  func @tpu_func(%arg0: tensor<2x6x8x6xsi8>) -> (tensor<2x8x6x20xsi8>, tensor<2x36x10x8xsi8>, tensor<2x36x8x18xsi8>, tensor<2x36x8x6xsi8>, tensor<2x36x4x3xsi8>) {
    %0 = "tpu.weight_file"() {filename = "movers_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.none"() : () -> none
    %2 = "tpu.input"(%arg0) {name = "input", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}} : (tensor<2x6x8x6xsi8>) -> tensor<2x6x8x6xsi8>
    %3 = "tpu.load_weight"(%0) {name = "c1_filter", storage = "INT8"} : (memref<10xf32>) -> tensor<36x6x3x3xf32>
    %4 = "tpu.load_weight"(%0) {name = "c1_bias", storage = "INT32"} : (memref<10xf32>) -> tensor<36xf32>
    %5 = "tpu.load_weight"(%0) {name = "c1_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<36xf32>
    %6 = "tpu.load_weight"(%0) {name = "c1_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<36xf32>
    %7 = "tpu.conv_2d"(%2, %3, %4, %1, %1, %5, %6) {name = "c1", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 0.000000e+00 : f32}, param = {dilation_h = 1 : i32, dilation_w = 1 : i32, group = 1 : i32, ins = [], is_dw = false, kernel_h = 3 : i32, kernel_w = 3 : i32, pad_value = 0 : i32, padding = "SAME", padding_b = 1 : i32, padding_l = 1 : i32, padding_r = 1 : i32, padding_t = 1 : i32, stride_h = 1 : i32, stride_w = 1 : i32, with_bias = true}, do_relu = false} : (tensor<2x6x8x6xsi8>, tensor<36x6x3x3xf32>, tensor<36xf32>, none, none, tensor<36xf32>, tensor<36xf32>) -> tensor<2x36x8x6xsi8>
    %8 = "tpu.pad"(%7) {name = "pad", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}, pads = [0 : i32, 0 : i32, 1 : i32, 2 : i32, 0 : i32, 0 : i32, 2 : i32, 1 : i32]} : (tensor<2x36x8x6xsi8>) -> tensor<2x36x11x9xsi8>
    %9 = "tpu.pad"(%7) {name = "pad_edge", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}, pads = [0 : i32, 0 : i32, 1 : i32, 1 : i32, 0 : i32, 0 : i32, 1 : i32, 1 : i32], mode = "edge"} : (tensor<2x36x8x6xsi8>) -> tensor<2x36x10x8xsi8>
    %10 = "tpu.crop"(%8) {name = "crop", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}, crop_offset = [0 : i32, 4 : i32, 1 : i32, 2 : i32]} : (tensor<2x36x11x9xsi8>) -> tensor<2x20x8x6xsi8>
    %11 = "tpu.permute"(%10) {name = "perm", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}, order = [0 : i32, 2 : i32, 3 : i32, 1 : i32]} : (tensor<2x20x8x6xsi8>) -> tensor<2x8x6x20xsi8>
    %12 = "tpu.reorg"(%7) {name = "reorg", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}, stride = 2 : i32} : (tensor<2x36x8x6xsi8>) -> tensor<2x144x4x3xsi8>
    %13 = "tpu.pixelshuffle"(%12) {name = "d2s", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}, mode = "DCR", upscale_factor = 2 : i32} : (tensor<2x144x4x3xsi8>) -> tensor<2x36x8x6xsi8>
    %14 = "tpu.tile"(%13) {name = "tile", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}, axis = 3 : i32, tiles = 3 : i32} : (tensor<2x36x8x6xsi8>) -> tensor<2x36x8x18xsi8>
    %15 = "tpu.reverse"(%14) {name = "rev", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}, axis = 2 : i32} : (tensor<2x36x8x18xsi8>) -> tensor<2x36x8x18xsi8>
    %16 = "tpu.shuffle_channel"(%15) {name = "shuf", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}, group = 4 : i32} : (tensor<2x36x8x18xsi8>) -> tensor<2x36x8x18xsi8>
    %17 = "tpu.relu"(%7) {name = "relu", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}} : (tensor<2x36x8x6xsi8>) -> tensor<2x36x8x6xsi8>
    %18 = "tpu.load_weight"(%0) {name = "avg_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %19 = "tpu.load_weight"(%0) {name = "avg_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %20 = "tpu.pool_avg_2d"(%7, %1, %1, %18, %19) {name = "avg", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 0.000000e+00 : f32}, param = {count_include_pad = false, kernel_h = 3 : i32, kernel_w = 3 : i32, pad_value = 0 : i32, padding_b = 0 : i32, padding_l = 1 : i32, padding_r = 0 : i32, padding_t = 1 : i32, stride_h = 2 : i32, stride_w = 2 : i32}, do_relu = false} : (tensor<2x36x8x6xsi8>, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<2x36x4x3xsi8>
    return %11, %9, %16, %17, %20 : tensor<2x8x6x20xsi8>, tensor<2x36x10x8xsi8>, tensor<2x36x8x18xsi8>, tensor<2x36x8x6xsi8>, tensor<2x36x4x3xsi8>
  }
}
