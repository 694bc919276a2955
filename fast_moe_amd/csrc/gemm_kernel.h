// Jagged ("grouped") GEMM for gfx950: out[rows of expert e] = A[gather] x B[e],
// bf16 or OCP-e4m3 operands, fp32 MFMA accumulation, fused bias / SiLU / SwiGLU
// epilogue.  Shared by gemm_bf16.hip and gemm_fp8.hip.
//
// Three kernels share the scheduler and the epilogue:
//
//   grouped_gemm_ring_kernel   the fast path.  Persistent (one block per CU), 256 x 256 tiles,
//       8 wavefronts.  Operand K-slices of 64 bytes per row travel global -> LDS with
//       global_load_lds_dwordx4 (no VGPR staging) into a ring of 32 KB slots; the ring runs
//       across tile boundaries, so the loads of the next tile are already under way while
//       the current tile's epilogue stores drain.  With few experts the ring takes all of
//       LDS (5 slots), slices are fetched in pairs as full 128-byte lines and the K loop is
//       a software pipeline of 8-MFMA blocks (see RingCfg); otherwise 4 slots, one slice at
//       a time, schedule tables in LDS.
//   grouped_gemm_stream_kernel experts with a handful of rows (the weights are streamed once
//       and that stream is the cost).  Persistent 64 x 256 tiles, 4 wavefronts, two blocks per
//       CU; a K-slice travels global -> registers -> LDS while the previous one is multiplied,
//       and the next tile's first slice is loaded before the current tile's epilogue, so the
//       weight stream does not stop at tile boundaries.
//   grouped_gemm_kernel        register-staged, double-buffered LDS; serves everything the
//       other two do not: arbitrary B strides and K / N tails (element loads), SiLU applied
//       to A on load, fp32 operands.
//
// e4m3 row-wise scales that are exact powers of two (GemmParams::scale_pow2) are handed to
// v_mfma_scale_f32_32x32x64_f8f6f4 as E8M0 codes of their reciprocals instead of being divided
// out in the epilogue (ring and streaming kernels; template parameter MSC).
//
// Mapping to the hardware
//   * LDS rows are XOR-swizzled in 16-byte chunks so that the ds_read_b128 of an MFMA
//     fragment is conflict free; for the ring kernel the swizzle is applied by permuting
//     which global chunk each lane fetches, because LDS-DMA lays lanes out linearly.
//   * The weights feed the MFMA "A" port and the activations the "B" port
//     (v_mfma_f32_32x32x16_bf16 / v_mfma_f32_32x32x64_f8f6f4), so a lane holds 4 consecutive
//     output columns of one output row per register quad; v_permlane32_swap pairs two
//     quads into 16 contiguous bytes for the store.
//   * Activation rows are gathered through row_index while loading (no [R, K] copy); rows
//     past the end of an expert segment re-read the tile's first row and are masked at the
//     store.
//   * Scheduling is on the device: the number of row tiles per expert comes from `offsets`
//     (wavefront prefix scan), so no max_seq_len and no host synchronisation are needed and
//     skewed or empty experts cost nothing.  Block ids are dealt round-robin to the 8 XCDs by
//     the hardware; id -> tile is remapped so that each XCD works on whole groups of tiles
//     (4 row tiles x all column tiles, what shares operands), which keeps them in its L2: the
//     paired ring deals the groups to the XCDs back and forth, the other kernels give every
//     XCD one contiguous range of the tile order.
//
// Files: gemm_params.h (launch parameters, helpers), gemm_epilogue.h, gemm_ring.h, gemm_stream.h,
// gemm_staged.h (the kernels), gemm_launch.h (kernel choice and launches).
#pragma once

#include "gemm_launch.h"
