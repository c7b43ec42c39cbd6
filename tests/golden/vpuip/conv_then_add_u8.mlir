// Written for these tests in the syntax the reference prints after lowering to VPUIP
// (compare tests/lit/NPU/conversion/passes/VPUIP2VPUMI37XX/nce_eltwise_37XX.mlir and nce_conv_37XX.mlir):
// DMA the input into CMX, a 3x3 quantized convolution in two variants, an eltwise add of the result with the
// input, DMA the sum out.
// RUN: vpux-opt --init-compiler="vpu-arch=VPUX37XX" --convert-VPUIP-to-VPUMI37XX %s

#NHWC = affine_map<(d0, d1, d2, d3) -> (d0, d2, d3, d1)>
!qIn = !quant.uniform<u8:f32, 2.000000e-02:128>
!qW = !quant.uniform<u8<0:254>:f32, 5.000000e-03:127>
!qMid = !quant.uniform<u8:f32, 5.000000e-02:121>
!qOut = !quant.uniform<u8:f32, 1.000000e-01:3>

module @mainModule {

  IE.CNNNetwork entryPoint : @convThenAdd inputsInfo : {
    DataInfo "input_0" : tensor<1x32x12x12xui8>
  } outputsInfo : {
    DataInfo "output_0" : tensor<1x32x12x12xui8>
  }

func.func @convThenAdd(%arg0: memref<1x32x12x12x!qIn, #NHWC, @DDR>, %arg1: memref<1x32x12x12x!qOut, #NHWC, @DDR>) -> memref<1x32x12x12x!qOut, #NHWC, @DDR> {
  %bar0 = VPURT.ConfigureBarrier<0> -> !VPURT.Barrier
  %bar1 = VPURT.ConfigureBarrier<1> -> !VPURT.Barrier
  %0 = VPURT.DeclareBuffer <CMX_NN> [0] <0> -> memref<1x32x12x12x!qIn, #NHWC, [@CMX_NN, 0]>
  %1 = VPURT.DeclareBuffer <CMX_NN> [0] <4608> -> memref<32x32x3x3x!qW, #NHWC, [@CMX_NN, 0]>
  %2 = VPURT.DeclareBuffer <CMX_NN> [0] <13824> -> memref<32x1x1x4xsi32, #NHWC, [@CMX_NN, 0]>
  %3 = VPURT.DeclareBuffer <CMX_NN> [0] <14336> -> memref<1x32x12x12x!qMid, #NHWC, [@CMX_NN, 0]>
  %4 = VPURT.DeclareBuffer <CMX_NN> [0] <18944> -> memref<1x32x12x12x!qOut, #NHWC, [@CMX_NN, 0]>
  %5 = VPURT.DeclareBuffer <DDR> <0> -> memref<32x32x3x3x!qW, #NHWC, @DDR>
  %6 = VPURT.DeclareBuffer <DDR> <9216> -> memref<32x1x1x4xsi32, #NHWC, @DDR>
  VPURT.Task updates(%bar0 : !VPURT.Barrier) {
    %10 = VPUIP.NNDMA {port = 0 : i64} inputs(%arg0 : memref<1x32x12x12x!qIn, #NHWC, @DDR>) outputs(%0 : memref<1x32x12x12x!qIn, #NHWC, [@CMX_NN, 0]>) -> memref<1x32x12x12x!qIn, #NHWC, [@CMX_NN, 0]>
  }
  VPURT.Task updates(%bar0 : !VPURT.Barrier) {
    %11 = VPUIP.NNDMA {port = 0 : i64} inputs(%5 : memref<32x32x3x3x!qW, #NHWC, @DDR>) outputs(%1 : memref<32x32x3x3x!qW, #NHWC, [@CMX_NN, 0]>) -> memref<32x32x3x3x!qW, #NHWC, [@CMX_NN, 0]>
  }
  VPURT.Task updates(%bar0 : !VPURT.Barrier) {
    %12 = VPUIP.NNDMA {port = 0 : i64} inputs(%6 : memref<32x1x1x4xsi32, #NHWC, @DDR>) outputs(%2 : memref<32x1x1x4xsi32, #NHWC, [@CMX_NN, 0]>) -> memref<32x1x1x4xsi32, #NHWC, [@CMX_NN, 0]>
  }
  VPURT.Task waits(%bar0 : !VPURT.Barrier) updates(%bar1 : !VPURT.Barrier) {
    %13 = VPUIP.NCEClusterTask {kernel_padding = #VPU.Padding<left = 1 : i64, right = 1 : i64, top = 1 : i64, bottom = 1 : i64>, kernel_size = [3, 3], kernel_strides = [1, 1], task_type = #VPUIP.nce_task_type<CONV>} input(%0 : memref<1x32x12x12x!qIn, #NHWC, [@CMX_NN, 0]>) weights(%1 : memref<32x32x3x3x!qW, #NHWC, [@CMX_NN, 0]>) weight_table(%2 : memref<32x1x1x4xsi32, #NHWC, [@CMX_NN, 0]>) parent_input(%0 : memref<1x32x12x12x!qIn, #NHWC, [@CMX_NN, 0]>) parent_output(%3 : memref<1x32x12x12x!qMid, #NHWC, [@CMX_NN, 0]>) outputs(%3 : memref<1x32x12x12x!qMid, #NHWC, [@CMX_NN, 0]>) -> memref<1x32x12x12x!qMid, #NHWC, [@CMX_NN, 0]> variants : {
      DPUTask {outEnd = [11, 5, 31], mpe_mode = #VPU.mpe_mode<CUBOID_16x16>, pad = #VPU.Padding<left = 1 : i64, right = 1 : i64, top = 1 : i64, bottom = 0 : i64>, outStart = [0, 0, 0]}
      DPUTask {outEnd = [11, 11, 31], mpe_mode = #VPU.mpe_mode<CUBOID_16x16>, pad = #VPU.Padding<left = 1 : i64, right = 1 : i64, top = 0 : i64, bottom = 1 : i64>, outStart = [0, 6, 0]}
    } PPE : {
      PPETask <LPRELU> {clamp_high = 255 : i64, clamp_low = 0 : i64, fp_prelu_alpha = 0.10000000149011612 : f64, lrelu_mult = 1638 : i64, lrelu_shift = 14 : i64}
    }
  }
  VPURT.Task waits(%bar1 : !VPURT.Barrier) {
    %14 = VPUIP.NCEClusterTask {activation_window_channel_length = 0 : i32, task_type = #VPUIP.nce_task_type<ELTWISE>} input(%3 : memref<1x32x12x12x!qMid, #NHWC, [@CMX_NN, 0]>) weights(%0 : memref<1x32x12x12x!qIn, #NHWC, [@CMX_NN, 0]>) parent_input(%3 : memref<1x32x12x12x!qMid, #NHWC, [@CMX_NN, 0]>) parent_output(%4 : memref<1x32x12x12x!qOut, #NHWC, [@CMX_NN, 0]>) outputs(%4 : memref<1x32x12x12x!qOut, #NHWC, [@CMX_NN, 0]>) -> memref<1x32x12x12x!qOut, #NHWC, [@CMX_NN, 0]> variants : {
      DPUTask {outEnd = [11, 11, 31], mpe_mode = #VPU.mpe_mode<CUBOID_8x16>, pad = #VPU.Padding<left = 0 : i64, right = 0 : i64, top = 0 : i64, bottom = 0 : i64>, outStart = [0, 0, 0]}
    } PPE : {
      PPETask <ADD> {clamp_high = 255 : i64, clamp_low = 3 : i64, in1_quant_mult = [20480], in2_quant_mult = [8192], lrelu_mult = 1 : i64, lrelu_shift = 0 : i64, quant_mult = [25600], quant_post_shift = 0 : i64, quant_scale = [1.000000e+00], quant_shift = [30]}
    }
  }
  VPURT.Task {
    %15 = VPUIP.NNDMA {port = 0 : i64} inputs(%4 : memref<1x32x12x12x!qOut, #NHWC, [@CMX_NN, 0]>) outputs(%arg1 : memref<1x32x12x12x!qOut, #NHWC, @DDR>) -> memref<1x32x12x12x!qOut, #NHWC, @DDR>
  }
  return %arg1 : memref<1x32x12x12x!qOut, #NHWC, @DDR>
}
}

// CHECK: func.func @convThenAdd
// CHECK: VPUMI37XX.DPUInvariant
