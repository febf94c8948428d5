// One mmt4d dispatch that reaches the MI355X plugin through a dynamic import.
// Not compiled in this repository (iree-compile is not part of it); it shows
// the operand order the plugin's imports expect, which is the order the
// reference's own lowering emits for iree_uk_mmt4d
// (compiler/src/iree/compiler/Codegen/Common/CPU/CPULowerToUKernels.cpp:252-274).
//
//   iree-compile --iree-hal-target-backends=llvm-cpu example.mlir -o example.vmfb
//   iree-run-module --device=local-sync \
//       --executable_plugin=libmi355x_uk_plugin.so \
//       --module=example.vmfb --function=mmt4d_i8 \
//       --input=4x8x32x16xi8=1 --input=4x8x32x16xi8=1
//
// Without `hal.import.bitcode` in fn_def_attrs the call is not resolved against
// the bundled microkernel bitcode but left as an import, which the runtime
// resolves by asking each loaded plugin (resolve() of mi355x_uk_plugin.c).
// Tiles are the gfx950 ones: M0 = N0 = 32, K0 = 16 for i8.

func.func @mmt4d_i8(%lhs : tensor<4x8x32x16xi8>, %rhs : tensor<4x8x32x16xi8>) -> tensor<4x4x32x32xi32> {
  %c1 = arith.constant 1 : index
  %acc = tensor.empty() : tensor<4x4x32x32xi32>
  %0 = flow.dispatch.region[%c1] -> (tensor<4x4x32x32xi32>) {
    %m = arith.constant 4 : index
    %n = arith.constant 4 : index
    %k = arith.constant 8 : index
    %m0 = arith.constant 32 : i32
    %n0 = arith.constant 32 : i32
    %k0 = arith.constant 16 : i32
    // IREE_UK_FLAG_MMT4D_TYPE_S8S8S32 (0x02) | ALLOW_GENERIC_FALLBACK_TILE_FUNCTION (0x200)
    %flags = arith.constant 514 : i32
    %1 = iree_codegen.ukernel.generic "mi355x_uk_mmt4d"
      ins(%lhs, %rhs : tensor<4x8x32x16xi8>, tensor<4x8x32x16xi8>)
      outs(%acc : tensor<4x4x32x32xi32>)
      (%m, %n, %k, %m0, %n0, %k0, %flags : index, index, index, i32, i32, i32, i32)
      fn_def_attrs {hal.import.fields = ["processor_data"]}
      strided_outer_dims(1) -> tensor<4x4x32x32xi32>
    flow.return %1 : tensor<4x4x32x32xi32>
  } count(%b0 : index) -> (index, index, index) {
    flow.return %b0, %b0, %b0 : index, index, index
  }
  return %0 : tensor<4x4x32x32xi32>
}
