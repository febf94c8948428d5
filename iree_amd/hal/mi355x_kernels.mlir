// hal.executable.source for iree_amd/hal/mi355x_kernels_gfx950.co: the gfx950
// mmt4d, pack, unpack and int4 dequantising matmul kernels as hand-written dispatches on a HIP device, after the
// reference's samples/custom_dispatch/hip/kernels/example.mlir:16-118.
// Written by iree_amd.hal_executable.mlir_source(); NOT compiled here (this
// build has no iree-compile).
//
// Every mmt4d export: bindings lhs (read only), rhs (read only), out; push constants
// M, N, K (outer tile counts), K0, flags (0x100 = accumulate), and for
// mi355x_mmt4d_unpack_* also out_rows, out_cols. The workload of a dispatch is
// (M, N, batch): batch = 1 for linalg.mmt4d, the batch size of a
// linalg.batch_mmt4d on dense operands (workgroup planes in y).

#rocm_gfx950_target = #hal.executable.target<"rocm", "rocm-hsaco-fb", {
  target_arch = "gfx950"
}>

hal.executable.source public @mi355x_mmt4d attributes {
  objects = #hal.executable.objects<{
    #rocm_gfx950_target = [
      #hal.executable.object<{path = "iree_amd/hal/mi355x_kernels_gfx950.co"}>
    ]
  }>
} {
  hal.executable.export public @mi355x_mmt4d_f16f16f32_t8 ordinal(0)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 163840 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 8) * (s1 ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_unpack_f16f16f32_t8 ordinal(1)
      layout(#hal.pipeline.layout<push_constants = 7, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 163840 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 8) * (s1 ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_f16f16f32_t4 ordinal(2)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 65536 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 4) * (s1 ceildiv 4))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_unpack_f16f16f32_t4 ordinal(3)
      layout(#hal.pipeline.layout<push_constants = 7, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 65536 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 4) * (s1 ceildiv 4))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_bf16bf16f32_t8 ordinal(4)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 163840 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 8) * (s1 ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_unpack_bf16bf16f32_t8 ordinal(5)
      layout(#hal.pipeline.layout<push_constants = 7, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 163840 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 8) * (s1 ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_bf16bf16f32_t4 ordinal(6)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 65536 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 4) * (s1 ceildiv 4))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_unpack_bf16bf16f32_t4 ordinal(7)
      layout(#hal.pipeline.layout<push_constants = 7, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 65536 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 4) * (s1 ceildiv 4))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_s8s8s32_t8 ordinal(8)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 163840 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 8) * (s1 ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_unpack_s8s8s32_t8 ordinal(9)
      layout(#hal.pipeline.layout<push_constants = 7, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 163840 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 8) * (s1 ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_s8s8s32_t4 ordinal(10)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 65536 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 4) * (s1 ceildiv 4))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_unpack_s8s8s32_t4 ordinal(11)
      layout(#hal.pipeline.layout<push_constants = 7, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 65536 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 4) * (s1 ceildiv 4))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_f8e4m3f8e4m3f32_t8 ordinal(12)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 163840 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 8) * (s1 ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_unpack_f8e4m3f8e4m3f32_t8 ordinal(13)
      layout(#hal.pipeline.layout<push_constants = 7, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 163840 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 8) * (s1 ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_f8e4m3f8e4m3f32_t4 ordinal(14)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 131072 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 4) * (s1 ceildiv 4))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_unpack_f8e4m3f8e4m3f32_t4 ordinal(15)
      layout(#hal.pipeline.layout<push_constants = 7, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 131072 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 4) * (s1 ceildiv 4))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_f32f32f32_t8 ordinal(16)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 131072 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 8) * (s1 ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_unpack_f32f32f32_t8 ordinal(17)
      layout(#hal.pipeline.layout<push_constants = 7, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 131072 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 8) * (s1 ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_f32f32f32_t4 ordinal(18)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 65536 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 4) * (s1 ceildiv 4))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  hal.executable.export public @mi355x_mmt4d_unpack_f32f32f32_t4 ordinal(19)
      layout(#hal.pipeline.layout<push_constants = 7, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 65536 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv 4) * (s1 ceildiv 4))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }
  // out[M][N] (+)= lhs[M][K] * rhs (packed); push constants M, N, K (elements), K0, flags; workload (M, N)
  // limits: M * K elements of lhs below 2 GiB, K a multiple of the matrix-core K extent (else nothing is written)
  hal.executable.export public @mi355x_matmul_packed_rhs_f16f16f32_t4x8 ordinal(20)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 73728 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index):
    %x = affine.apply affine_map<()[s0, s1] -> (((s0 ceildiv 32) ceildiv 4) * ((s1 ceildiv 32) ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // out[M][N] (+)= lhs[M][K] * rhs (packed); push constants M, N, K (elements), K0, flags; workload (M, N)
  // limits: M * K elements of lhs below 2 GiB, K a multiple of the matrix-core K extent (else nothing is written)
  hal.executable.export public @mi355x_matmul_packed_rhs_f16f16f32_t8x8 ordinal(21)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 163840 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index):
    %x = affine.apply affine_map<()[s0, s1] -> (((s0 ceildiv 32) ceildiv 8) * ((s1 ceildiv 32) ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // out[M][N] (+)= lhs[M][K] * rhs (packed); push constants M, N, K (elements), K0, flags; workload (M, N)
  // limits: M * K elements of lhs below 2 GiB, K a multiple of the matrix-core K extent (else nothing is written)
  hal.executable.export public @mi355x_matmul_packed_rhs_bf16bf16f32_t4x8 ordinal(22)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 73728 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index):
    %x = affine.apply affine_map<()[s0, s1] -> (((s0 ceildiv 32) ceildiv 4) * ((s1 ceildiv 32) ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // out[M][N] (+)= lhs[M][K] * rhs (packed); push constants M, N, K (elements), K0, flags; workload (M, N)
  // limits: M * K elements of lhs below 2 GiB, K a multiple of the matrix-core K extent (else nothing is written)
  hal.executable.export public @mi355x_matmul_packed_rhs_bf16bf16f32_t8x8 ordinal(23)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 163840 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index):
    %x = affine.apply affine_map<()[s0, s1] -> (((s0 ceildiv 32) ceildiv 8) * ((s1 ceildiv 32) ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // out[M][N] (+)= lhs[M][K] * rhs (packed); push constants M, N, K (elements), K0, flags; workload (M, N)
  // limits: M * K elements of lhs below 2 GiB, K a multiple of the matrix-core K extent (else nothing is written)
  hal.executable.export public @mi355x_matmul_packed_rhs_s8s8s32_t4x8 ordinal(24)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 73728 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index):
    %x = affine.apply affine_map<()[s0, s1] -> (((s0 ceildiv 32) ceildiv 4) * ((s1 ceildiv 32) ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // out[M][N] (+)= lhs[M][K] * rhs (packed); push constants M, N, K (elements), K0, flags; workload (M, N)
  // limits: M * K elements of lhs below 2 GiB, K a multiple of the matrix-core K extent (else nothing is written)
  hal.executable.export public @mi355x_matmul_packed_rhs_s8s8s32_t8x8 ordinal(25)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 131072 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index):
    %x = affine.apply affine_map<()[s0, s1] -> (((s0 ceildiv 32) ceildiv 8) * ((s1 ceildiv 32) ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // out[M][N] (+)= lhs[M][K] * rhs (packed); push constants M, N, K (elements), K0, flags; workload (M, N)
  // limits: M * K elements of lhs below 2 GiB, K a multiple of the matrix-core K extent (else nothing is written)
  hal.executable.export public @mi355x_matmul_packed_rhs_s8s8s32_k64_t4x8 ordinal(26)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 73728 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index):
    %x = affine.apply affine_map<()[s0, s1] -> (((s0 ceildiv 32) ceildiv 4) * ((s1 ceildiv 32) ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // out[M][N] (+)= lhs[M][K] * rhs (packed); push constants M, N, K (elements), K0, flags; workload (M, N)
  // limits: M * K elements of lhs below 2 GiB, K a multiple of the matrix-core K extent (else nothing is written)
  hal.executable.export public @mi355x_matmul_packed_rhs_s8s8s32_k64_t8x8 ordinal(27)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 163840 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index):
    %x = affine.apply affine_map<()[s0, s1] -> (((s0 ceildiv 32) ceildiv 8) * ((s1 ceildiv 32) ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // out[M][N] (+)= lhs[M][K] * rhs (packed); push constants M, N, K (elements), K0, flags; workload (M, N)
  // limits: M * K elements of lhs below 2 GiB, K a multiple of the matrix-core K extent (else nothing is written)
  hal.executable.export public @mi355x_matmul_packed_rhs_f8e4m3f8e4m3f32_t4x8 ordinal(28)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 73728 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index):
    %x = affine.apply affine_map<()[s0, s1] -> (((s0 ceildiv 32) ceildiv 4) * ((s1 ceildiv 32) ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // out[M][N] (+)= lhs[M][K] * rhs (packed); push constants M, N, K (elements), K0, flags; workload (M, N)
  // limits: M * K elements of lhs below 2 GiB, K a multiple of the matrix-core K extent (else nothing is written)
  hal.executable.export public @mi355x_matmul_packed_rhs_f8e4m3f8e4m3f32_t8x8 ordinal(29)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 163840 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index):
    %x = affine.apply affine_map<()[s0, s1] -> (((s0 ceildiv 32) ceildiv 8) * ((s1 ceildiv 32) ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // out[M][N] (+)= lhs[M][K] * rhs (packed); push constants M, N, K (elements), K0, flags; workload (M, N)
  // limits: M * K elements of lhs below 2 GiB, K a multiple of the matrix-core K extent (else nothing is written)
  hal.executable.export public @mi355x_matmul_packed_rhs_f32f32f32_t4x8 ordinal(30)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 73728 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index):
    %x = affine.apply affine_map<()[s0, s1] -> (((s0 ceildiv 32) ceildiv 4) * ((s1 ceildiv 32) ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // out[M][N] (+)= lhs[M][K] * rhs (packed); push constants M, N, K (elements), K0, flags; workload (M, N)
  // limits: M * K elements of lhs below 2 GiB, K a multiple of the matrix-core K extent (else nothing is written)
  hal.executable.export public @mi355x_matmul_packed_rhs_f32f32f32_t8x8 ordinal(31)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index],
    workgroup_local_memory = 131072 : index
  } {
  ^bb0(%device: !hal.device, %m: index, %n: index):
    %x = affine.apply affine_map<()[s0, s1] -> (((s0 ceildiv 32) ceildiv 8) * ((s1 ceildiv 32) ceildiv 8))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // pack: in = matrix, out = tiles; push constants size0, size1, tile0, tile1, padding; workload (size0, size1, tile0, tile1)
  // any tile size, no transposes; power-of-two tiles whose rows are whole 16-byte chunks stream 16-byte chunks, others move single elements
  hal.executable.export public @mi355x_pack_8bit ordinal(32)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index]
  } {
  ^bb0(%device: !hal.device, %size0: index, %size1: index, %tile0: index, %tile1: index):
    %c1 = arith.constant 1 : index
    %c16 = arith.constant 16 : index
    %c32 = arith.constant 32 : index
    %bytes = arith.constant 1 : index
    %o0 = arith.ceildivui %size0, %tile0 : index
    %rows = arith.muli %o0, %tile0 : index
    %o1 = arith.ceildivui %size1, %tile1 : index
    %cols = arith.muli %o1, %tile1 : index
    %row_bytes = arith.muli %cols, %bytes : index
    %chunks = arith.ceildivui %row_bytes, %c16 : index
    %bx = arith.ceildivui %chunks, %c32 : index
    %by = arith.ceildivui %rows, %c16 : index
    %x = arith.muli %bx, %by : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // pack: in = matrix, out = tiles; push constants size0, size1, tile0, tile1, padding; workload (size0, size1, tile0, tile1)
  // any tile size, no transposes; power-of-two tiles whose rows are whole 16-byte chunks stream 16-byte chunks, others move single elements
  hal.executable.export public @mi355x_pack_16bit ordinal(33)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index]
  } {
  ^bb0(%device: !hal.device, %size0: index, %size1: index, %tile0: index, %tile1: index):
    %c1 = arith.constant 1 : index
    %c16 = arith.constant 16 : index
    %c32 = arith.constant 32 : index
    %bytes = arith.constant 2 : index
    %o0 = arith.ceildivui %size0, %tile0 : index
    %rows = arith.muli %o0, %tile0 : index
    %o1 = arith.ceildivui %size1, %tile1 : index
    %cols = arith.muli %o1, %tile1 : index
    %row_bytes = arith.muli %cols, %bytes : index
    %chunks = arith.ceildivui %row_bytes, %c16 : index
    %bx = arith.ceildivui %chunks, %c32 : index
    %by = arith.ceildivui %rows, %c16 : index
    %x = arith.muli %bx, %by : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // pack: in = matrix, out = tiles; push constants size0, size1, tile0, tile1, padding; workload (size0, size1, tile0, tile1)
  // any tile size, no transposes; power-of-two tiles whose rows are whole 16-byte chunks stream 16-byte chunks, others move single elements
  hal.executable.export public @mi355x_pack_32bit ordinal(34)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index]
  } {
  ^bb0(%device: !hal.device, %size0: index, %size1: index, %tile0: index, %tile1: index):
    %c1 = arith.constant 1 : index
    %c16 = arith.constant 16 : index
    %c32 = arith.constant 32 : index
    %bytes = arith.constant 4 : index
    %o0 = arith.ceildivui %size0, %tile0 : index
    %rows = arith.muli %o0, %tile0 : index
    %o1 = arith.ceildivui %size1, %tile1 : index
    %cols = arith.muli %o1, %tile1 : index
    %row_bytes = arith.muli %cols, %bytes : index
    %chunks = arith.ceildivui %row_bytes, %c16 : index
    %bx = arith.ceildivui %chunks, %c32 : index
    %by = arith.ceildivui %rows, %c16 : index
    %x = arith.muli %bx, %by : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // unpack: in = tiles, out = matrix; push constants size0, size1, tile0, tile1; workload (size0, size1, tile0, tile1)
  // any tile size, no transposes; power-of-two tiles whose rows are whole 16-byte chunks stream 16-byte chunks, others move single elements
  hal.executable.export public @mi355x_unpack_16bit ordinal(35)
      layout(#hal.pipeline.layout<push_constants = 4, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index]
  } {
  ^bb0(%device: !hal.device, %size0: index, %size1: index, %tile0: index, %tile1: index):
    %c1 = arith.constant 1 : index
    %c16 = arith.constant 16 : index
    %c32 = arith.constant 32 : index
    %bytes = arith.constant 2 : index
    %row_bytes = arith.muli %size1, %bytes : index
    %chunks = arith.ceildivui %row_bytes, %c16 : index
    %bx = arith.ceildivui %chunks, %c32 : index
    %by = arith.ceildivui %size0, %c16 : index
    %x = arith.muli %bx, %by : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // unpack: in = tiles, out = matrix; push constants size0, size1, tile0, tile1; workload (size0, size1, tile0, tile1)
  // any tile size, no transposes; power-of-two tiles whose rows are whole 16-byte chunks stream 16-byte chunks, others move single elements
  hal.executable.export public @mi355x_unpack_32bit ordinal(36)
      layout(#hal.pipeline.layout<push_constants = 4, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index]
  } {
  ^bb0(%device: !hal.device, %size0: index, %size1: index, %tile0: index, %tile1: index):
    %c1 = arith.constant 1 : index
    %c16 = arith.constant 16 : index
    %c32 = arith.constant 32 : index
    %bytes = arith.constant 4 : index
    %row_bytes = arith.muli %size1, %bytes : index
    %chunks = arith.ceildivui %row_bytes, %c16 : index
    %bx = arith.ceildivui %chunks, %c32 : index
    %by = arith.ceildivui %size0, %c16 : index
    %x = arith.muli %bx, %by : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // pack: in = matrix, out = tiles, tiles of tile0 rows x tile1 columns stored column by column; push constants size0, size1, tile0, tile1, padding; workload (size0, size1, tile0, tile1)
  // any tile size; power-of-two tiles with tile0 * 1 >= 16 move 16-byte chunks, others single elements
  hal.executable.export public @mi355x_pack_transpose_8bit ordinal(37)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index]
  } {
  ^bb0(%device: !hal.device, %size0: index, %size1: index, %tile0: index, %tile1: index):
    %c1 = arith.constant 1 : index
    %c16 = arith.constant 16 : index
    %c64 = arith.constant 64 : index
    %bytes = arith.constant 1 : index
    %o0 = arith.ceildivui %size0, %tile0 : index
    %tile_bytes = arith.muli %tile0, %bytes : index
    %per_tile = arith.ceildivui %tile_bytes, %c16 : index
    %groups = arith.muli %o0, %per_tile : index
    %o1 = arith.ceildivui %size1, %tile1 : index
    %cols = arith.muli %o1, %tile1 : index
    %bx = arith.ceildivui %cols, %c64 : index
    %by = arith.ceildivui %groups, %c16 : index
    %x = arith.muli %bx, %by : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // pack: in = matrix, out = tiles, tiles of tile0 rows x tile1 columns stored column by column; push constants size0, size1, tile0, tile1, padding; workload (size0, size1, tile0, tile1)
  // any tile size; power-of-two tiles with tile0 * 2 >= 16 move 16-byte chunks, others single elements
  hal.executable.export public @mi355x_pack_transpose_16bit ordinal(38)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index]
  } {
  ^bb0(%device: !hal.device, %size0: index, %size1: index, %tile0: index, %tile1: index):
    %c1 = arith.constant 1 : index
    %c16 = arith.constant 16 : index
    %c64 = arith.constant 64 : index
    %bytes = arith.constant 2 : index
    %o0 = arith.ceildivui %size0, %tile0 : index
    %tile_bytes = arith.muli %tile0, %bytes : index
    %per_tile = arith.ceildivui %tile_bytes, %c16 : index
    %groups = arith.muli %o0, %per_tile : index
    %o1 = arith.ceildivui %size1, %tile1 : index
    %cols = arith.muli %o1, %tile1 : index
    %bx = arith.ceildivui %cols, %c64 : index
    %by = arith.ceildivui %groups, %c16 : index
    %x = arith.muli %bx, %by : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // pack: in = matrix, out = tiles, tiles of tile0 rows x tile1 columns stored column by column; push constants size0, size1, tile0, tile1, padding; workload (size0, size1, tile0, tile1)
  // any tile size; power-of-two tiles with tile0 * 4 >= 16 move 16-byte chunks, others single elements
  hal.executable.export public @mi355x_pack_transpose_32bit ordinal(39)
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index]
  } {
  ^bb0(%device: !hal.device, %size0: index, %size1: index, %tile0: index, %tile1: index):
    %c1 = arith.constant 1 : index
    %c16 = arith.constant 16 : index
    %c64 = arith.constant 64 : index
    %bytes = arith.constant 4 : index
    %o0 = arith.ceildivui %size0, %tile0 : index
    %tile_bytes = arith.muli %tile0, %bytes : index
    %per_tile = arith.ceildivui %tile_bytes, %c16 : index
    %groups = arith.muli %o0, %per_tile : index
    %o1 = arith.ceildivui %size1, %tile1 : index
    %cols = arith.muli %o1, %tile1 : index
    %bx = arith.ceildivui %cols, %c64 : index
    %by = arith.ceildivui %groups, %c16 : index
    %x = arith.muli %bx, %by : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // unpack: in = tiles, out = matrix, tiles of tile0 rows x tile1 columns stored column by column; push constants size0, size1, tile0, tile1; workload (size0, size1, tile0, tile1)
  // any tile size; power-of-two tiles with tile0 * 2 >= 16 move 16-byte chunks, others single elements
  hal.executable.export public @mi355x_unpack_transpose_16bit ordinal(40)
      layout(#hal.pipeline.layout<push_constants = 4, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index]
  } {
  ^bb0(%device: !hal.device, %size0: index, %size1: index, %tile0: index, %tile1: index):
    %c1 = arith.constant 1 : index
    %c16 = arith.constant 16 : index
    %c64 = arith.constant 64 : index
    %bytes = arith.constant 2 : index
    %o0 = arith.ceildivui %size0, %tile0 : index
    %tile_bytes = arith.muli %tile0, %bytes : index
    %per_tile = arith.ceildivui %tile_bytes, %c16 : index
    %groups = arith.muli %o0, %per_tile : index
    %bx = arith.ceildivui %size1, %c64 : index
    %by = arith.ceildivui %groups, %c16 : index
    %x = arith.muli %bx, %by : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // unpack: in = tiles, out = matrix, tiles of tile0 rows x tile1 columns stored column by column; push constants size0, size1, tile0, tile1; workload (size0, size1, tile0, tile1)
  // any tile size; power-of-two tiles with tile0 * 4 >= 16 move 16-byte chunks, others single elements
  hal.executable.export public @mi355x_unpack_transpose_32bit ordinal(41)
      layout(#hal.pipeline.layout<push_constants = 4, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [256 : index, 1 : index, 1 : index]
  } {
  ^bb0(%device: !hal.device, %size0: index, %size1: index, %tile0: index, %tile1: index):
    %c1 = arith.constant 1 : index
    %c16 = arith.constant 16 : index
    %c64 = arith.constant 64 : index
    %bytes = arith.constant 4 : index
    %o0 = arith.ceildivui %size0, %tile0 : index
    %tile_bytes = arith.muli %tile0, %bytes : index
    %per_tile = arith.ceildivui %tile_bytes, %c16 : index
    %groups = arith.muli %o0, %per_tile : index
    %bx = arith.ceildivui %size1, %c64 : index
    %by = arith.ceildivui %groups, %c16 : index
    %x = arith.muli %bx, %by : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // out[M][N] f16 = x[M][4096] f16 * int4 weights (tiled), groups of 128: f16 scales [N][32], packed uint4 zero points [N][32]
  // push constants M, N; workload (N); limits: 1 <= M <= 16, N a multiple of 32 (else nothing is written)
  hal.executable.export public @mi355x_dequant_matmul_i4_k4096_g128_r16 ordinal(42)
      layout(#hal.pipeline.layout<push_constants = 2, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer, ReadOnly>,
            <3, storage_buffer, ReadOnly>,
            <4, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [512 : index, 1 : index, 1 : index],
    workgroup_local_memory = 131072 : index
  } {
  ^bb0(%device: !hal.device, %n: index):
    %c1 = arith.constant 1 : index
    %c32 = arith.constant 32 : index
    %cmax = arith.constant 256 : index
    %tiles = arith.divui %n, %c32 : index
    %x = arith.minui %tiles, %cmax : index
    hal.return %x, %c1, %c1 : index, index, index
  }
  // out[M][N] f16 = x[M][4096] f16 * int4 weights (tiled), groups of 128: f16 scales [N][32], packed uint4 zero points [N][32]
  // push constants M, N; workload (N); limits: 1 <= M <= 32, N a multiple of 32 (else nothing is written)
  hal.executable.export public @mi355x_dequant_matmul_i4_k4096_g128_r32 ordinal(43)
      layout(#hal.pipeline.layout<push_constants = 2, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer, ReadOnly>,
            <3, storage_buffer, ReadOnly>,
            <4, storage_buffer>
        ]>
      ]>) attributes {
    workgroup_size = [512 : index, 1 : index, 1 : index],
    workgroup_local_memory = 131072 : index
  } {
  ^bb0(%device: !hal.device, %n: index):
    %c1 = arith.constant 1 : index
    %c32 = arith.constant 32 : index
    %cmax = arith.constant 256 : index
    %tiles = arith.divui %n, %c32 : index
    %x = arith.minui %tiles, %cmax : index
    hal.return %x, %c1, %c1 : index, index, index
  }
}

// A dispatch site (f16, 4096^3: M = N = 128 outer tiles, K = 512 tiles of K0 = 8):
//   %out = flow.dispatch @mi355x_mmt4d::@mi355x_mmt4d_f16f16f32_t8[%c128, %c128, %c1](
//       %c128_i32, %c128_i32, %c512_i32, %c8_i32, %c0_i32, %lhs, %rhs)
//     : (i32, i32, i32, i32, i32, tensor<128x512x32x8xf16>, tensor<128x512x32x8xf16>)
//       -> tensor<128x128x32x32xf32>
// (primitive operands come first and must be i32, example.mlir:128-140; with
// the accumulate flag the result is tied to a third tensor operand: `-> %acc`.)
