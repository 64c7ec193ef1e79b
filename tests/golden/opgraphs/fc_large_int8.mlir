module {
  func @tpu_func(%arg0: tensor<201x512xf32>) -> tensor<201x23501xf32> {
    %0 = "tpu.weight_file"() {filename = "fc_large_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 8.650300e-01 : f32}} : (tensor<201x512xf32>) -> tensor<201x512xf32>
    %2 = "tpu.none"() : () -> none
    %3 = "tpu.load_weight"(%0) {name = "filter_quant", storage = "INT8"} : (memref<10xf32>) -> tensor<23501x512xf32>
    %q0 = "tpu.load_weight"(%0) {name = "fc_large_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q1 = "tpu.load_weight"(%0) {name = "fc_large_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q2 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 0x4313F8C4 : f32, name = "data_quant_i8"} : (tensor<201x512xf32>) -> tensor<201x512xsi8>
    %5 = "tpu.fully_connected"(%q2, %3, %2, %2, %2, %q0, %q1) {name = "fc_large", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 1.101170e+00 : f32}} : (tensor<201x512xsi8>, tensor<23501x512xf32>, none, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<201x23501xsi8>
    %q3 = "tpu.quant"(%5) {from = "INT8", to = "NONE", scale = 8.602890e-03 : f32, name = "fc_large_dequant"} : (tensor<201x23501xsi8>) -> tensor<201x23501xf32>
    return %q3 : tensor<201x23501xf32>
  }
}
