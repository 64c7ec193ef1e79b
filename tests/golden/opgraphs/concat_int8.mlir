module {
  func @tpu_func(%arg0: tensor<32x32x32x32xf32>) -> (tensor<96x32x32x32xf32>, tensor<32x96x32x32xf32>, tensor<32x32x96x32xf32>, tensor<32x32x32x96xf32>, tensor<64x32x1024xf32>, tensor<32x64x1024xf32>, tensor<32x32x2048xf32>, tensor<2048x1024xf32>, tensor<1024x2048xf32>) {
    %q0 = "tpu.weight_file"() {filename = "concat_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 3.068540e+00 : f32}} : (tensor<32x32x32x32xf32>) -> tensor<32x32x32x32xf32>
    %2 = "tpu.none"() : () -> none
    %q19 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 0x4226DAC6 : f32, name = "data_quant_i8"} : (tensor<32x32x32x32xf32>) -> tensor<32x32x32x32xsi8>
    %3 = "tpu.permute"(%q19) {name = "permute_1023", order = [1 : i32, 0 : i32, 2 : i32, 3 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 3.068540e+00 : f32}} : (tensor<32x32x32x32xsi8>) -> tensor<32x32x32x32xsi8>
    %5 = "tpu.reshape"(%3) {name = "reshape_1"} : (tensor<32x32x32x32xsi8>) -> tensor<32x32x1024xsi8>
    %8 = "tpu.reshape"(%3) {name = "reshape_4"} : (tensor<32x32x32x32xsi8>) -> tensor<1024x1024xsi8>
    %q1 = "tpu.load_weight"(%q0) {name = "concat4_0_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<3xf32>
    %q2 = "tpu.load_weight"(%q0) {name = "concat4_0_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<3xf32>
    %9 = "tpu.concat"(%q19, %q19, %q19, %2, %2, %q1, %q2) {axis = 0 : i32, name = "concat4_0", do_relu = true, quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 3.328160e+00 : f32}} : (tensor<32x32x32x32xsi8>, tensor<32x32x32x32xsi8>, tensor<32x32x32x32xsi8>, none, none, tensor<3xf32>, tensor<3xf32>) -> tensor<96x32x32x32xsi8>
    %q3 = "tpu.load_weight"(%q0) {name = "concat4_1_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<3xf32>
    %q4 = "tpu.load_weight"(%q0) {name = "concat4_1_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<3xf32>
    %10 = "tpu.concat"(%q19, %q19, %q19, %2, %2, %q3, %q4) {axis = 1 : i32, name = "concat4_1", do_relu = true, quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 3.901580e+00 : f32}} : (tensor<32x32x32x32xsi8>, tensor<32x32x32x32xsi8>, tensor<32x32x32x32xsi8>, none, none, tensor<3xf32>, tensor<3xf32>) -> tensor<32x96x32x32xsi8>
    %q5 = "tpu.load_weight"(%q0) {name = "concat4_2_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<3xf32>
    %q6 = "tpu.load_weight"(%q0) {name = "concat4_2_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<3xf32>
    %11 = "tpu.concat"(%q19, %q19, %q19, %2, %2, %q5, %q6) {axis = 2 : i32, name = "concat4_2", do_relu = false, quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 2.174060e+00 : f32}} : (tensor<32x32x32x32xsi8>, tensor<32x32x32x32xsi8>, tensor<32x32x32x32xsi8>, none, none, tensor<3xf32>, tensor<3xf32>) -> tensor<32x32x96x32xsi8>
    %q7 = "tpu.load_weight"(%q0) {name = "concat4_3_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<3xf32>
    %q8 = "tpu.load_weight"(%q0) {name = "concat4_3_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<3xf32>
    %12 = "tpu.concat"(%q19, %q19, %q19, %2, %2, %q7, %q8) {axis = 3 : i32, name = "concat4_3", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 2.300750e+00 : f32}} : (tensor<32x32x32x32xsi8>, tensor<32x32x32x32xsi8>, tensor<32x32x32x32xsi8>, none, none, tensor<3xf32>, tensor<3xf32>) -> tensor<32x32x32x96xsi8>
    %q9 = "tpu.load_weight"(%q0) {name = "concat3_0_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<2xf32>
    %q10 = "tpu.load_weight"(%q0) {name = "concat3_0_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<2xf32>
    %13 = "tpu.concat"(%5, %5, %2, %2, %q9, %q10) {axis = 0 : i32, name = "concat3_0", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 1.733850e+00 : f32}} : (tensor<32x32x1024xsi8>, tensor<32x32x1024xsi8>, none, none, tensor<2xf32>, tensor<2xf32>) -> tensor<64x32x1024xsi8>
    %q11 = "tpu.load_weight"(%q0) {name = "concat3_1_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<2xf32>
    %q12 = "tpu.load_weight"(%q0) {name = "concat3_1_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<2xf32>
    %14 = "tpu.concat"(%5, %5, %2, %2, %q11, %q12) {axis = 1 : i32, name = "concat3_1", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 2.394240e+00 : f32}} : (tensor<32x32x1024xsi8>, tensor<32x32x1024xsi8>, none, none, tensor<2xf32>, tensor<2xf32>) -> tensor<32x64x1024xsi8>
    %q13 = "tpu.load_weight"(%q0) {name = "concat3_2_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<2xf32>
    %q14 = "tpu.load_weight"(%q0) {name = "concat3_2_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<2xf32>
    %15 = "tpu.concat"(%5, %5, %2, %2, %q13, %q14) {axis = 2 : i32, name = "concat3_2", do_relu = true, quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 3.770960e+00 : f32}} : (tensor<32x32x1024xsi8>, tensor<32x32x1024xsi8>, none, none, tensor<2xf32>, tensor<2xf32>) -> tensor<32x32x2048xsi8>
    %q15 = "tpu.load_weight"(%q0) {name = "concat2_0_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<2xf32>
    %q16 = "tpu.load_weight"(%q0) {name = "concat2_0_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<2xf32>
    %16 = "tpu.concat"(%8, %8, %2, %2, %q15, %q16) {axis = 0 : i32, name = "concat2_0", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 1.076530e+00 : f32}} : (tensor<1024x1024xsi8>, tensor<1024x1024xsi8>, none, none, tensor<2xf32>, tensor<2xf32>) -> tensor<2048x1024xsi8>
    %q17 = "tpu.load_weight"(%q0) {name = "concat2_1_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<2xf32>
    %q18 = "tpu.load_weight"(%q0) {name = "concat2_1_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<2xf32>
    %17 = "tpu.concat"(%8, %8, %2, %2, %q17, %q18) {axis = 1 : i32, name = "concat2_1", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 1.061860e+00 : f32}} : (tensor<1024x1024xsi8>, tensor<1024x1024xsi8>, none, none, tensor<2xf32>, tensor<2xf32>) -> tensor<1024x2048xsi8>
    %q20 = "tpu.quant"(%9) {from = "INT8", to = "NONE", scale = 2.600125e-02 : f32, name = "concat4_0_dequant"} : (tensor<96x32x32x32xsi8>) -> tensor<96x32x32x32xf32>
    %q21 = "tpu.quant"(%10) {from = "INT8", to = "NONE", scale = 0x3CF9B37D : f32, name = "concat4_1_dequant"} : (tensor<32x96x32x32xsi8>) -> tensor<32x96x32x32xf32>
    %q22 = "tpu.quant"(%11) {from = "INT8", to = "NONE", scale = 0x3C8B23CD : f32, name = "concat4_2_dequant"} : (tensor<32x32x96x32xsi8>) -> tensor<32x32x96x32xf32>
    %q23 = "tpu.quant"(%12) {from = "INT8", to = "NONE", scale = 1.797461e-02 : f32, name = "concat4_3_dequant"} : (tensor<32x32x32x96xsi8>) -> tensor<32x32x32x96xf32>
    %q24 = "tpu.quant"(%13) {from = "INT8", to = "NONE", scale = 0x3C5DEECC : f32, name = "concat3_0_dequant"} : (tensor<64x32x1024xsi8>) -> tensor<64x32x1024xf32>
    %q25 = "tpu.quant"(%14) {from = "INT8", to = "NONE", scale = 1.870500e-02 : f32, name = "concat3_1_dequant"} : (tensor<32x64x1024xsi8>) -> tensor<32x64x1024xf32>
    %q26 = "tpu.quant"(%15) {from = "INT8", to = "NONE", scale = 0x3CF15769 : f32, name = "concat3_2_dequant"} : (tensor<32x32x2048xsi8>) -> tensor<32x32x2048xf32>
    %q27 = "tpu.quant"(%16) {from = "INT8", to = "NONE", scale = 0x3C09CBBC : f32, name = "concat2_0_dequant"} : (tensor<2048x1024xsi8>) -> tensor<2048x1024xf32>
    %q28 = "tpu.quant"(%17) {from = "INT8", to = "NONE", scale = 8.295781e-03 : f32, name = "concat2_1_dequant"} : (tensor<1024x2048xsi8>) -> tensor<1024x2048xf32>
    return %q20, %q21, %q22, %q23, %q24, %q25, %q26, %q27, %q28 : tensor<96x32x32x32xf32>, tensor<32x96x32x32xf32>, tensor<32x32x96x32xf32>, tensor<32x32x32x96xf32>, tensor<64x32x1024xf32>, tensor<32x64x1024xf32>, tensor<32x32x2048xf32>, tensor<2048x1024xf32>, tensor<1024x2048xf32>
  }
}
