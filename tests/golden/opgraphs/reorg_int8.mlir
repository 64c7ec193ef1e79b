module {
  func @tpu_func(%arg0: tensor<4x64x68x120xf32>) -> tensor<4x256x34x60xf32> {
    %0 = "tpu.weight_file"() {filename = "reorg_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 3.152670e+00 : f32}} : (tensor<4x64x68x120xf32>) -> tensor<4x64x68x120xf32>
    %q0 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 4.060051e+01 : f32, name = "data_quant_i8"} : (tensor<4x64x68x120xf32>) -> tensor<4x64x68x120xsi8>
    %2 = "tpu.reorg"(%q0) {name = "reorg", quant = {mode = "INT8", param_type = "NONE", threshold = 3.152670e+00 : f32}, stride = 2 : i32} : (tensor<4x64x68x120xsi8>) -> tensor<4x256x34x60xsi8>
    %q1 = "tpu.quant"(%2) {from = "INT8", to = "NONE", scale = 0x3CC9C558 : f32, name = "reorg_dequant"} : (tensor<4x256x34x60xsi8>) -> tensor<4x256x34x60xf32>
    return %q1 : tensor<4x256x34x60xf32>
  }
}
