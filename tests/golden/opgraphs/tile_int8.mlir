module {
  func @tpu_func(%arg0: tensor<1x256x1x1xf32>) -> tensor<1x256x31x31xf32> {
    %0 = "tpu.weight_file"() {filename = "tile_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "input", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 8.344300e-01 : f32}} : (tensor<1x256x1x1xf32>) -> tensor<1x256x1x1xf32>
    %2 = "tpu.none"() : () -> none
    %q0 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 0x431965EC : f32, name = "input_quant_i8"} : (tensor<1x256x1x1xf32>) -> tensor<1x256x1x1xsi8>
    %3 = "tpu.tile"(%q0) {name = "tile_h", quant = {mode = "INT8", param_type = "NONE", threshold = 8.344300e-01 : f32}, axis = 2 : i32, tiles = 31 : i32} : (tensor<1x256x1x1xsi8>) -> tensor<1x256x31x1xsi8>
    %4 = "tpu.tile"(%3) {name = "tile_w", quant = {mode = "INT8", param_type = "NONE", threshold = 8.344300e-01 : f32}, axis = 3 : i32, tiles = 31 : i32} : (tensor<1x256x31x1xsi8>) -> tensor<1x256x31x31xsi8>
    %q1 = "tpu.quant"(%4) {from = "INT8", to = "NONE", scale = 6.518984e-03 : f32, name = "tile_w_dequant"} : (tensor<1x256x31x31xsi8>) -> tensor<1x256x31x31xf32>
    return %q1 : tensor<1x256x31x31xf32>
  }
}
