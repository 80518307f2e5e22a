// Numbers that the product kernels (gemm.hip) and the rule for K ranges (engine.hip) share.
#pragma once

// The kernel with 32 x 32 tiles and the rows through LDS (gemm_bf16_rows32) takes steps of more
// than KAPPAI_ROWS32_MIN_ROWS and up to KAPPAI_ROWS32_MAX_ROWS rows.  Below, the kernels with
// 16 x 16 tiles are as fast or faster (up to 24 rows they read the rows of A straight from L2);
// above, the block kernels.  Measured on one box, decode steps of the LFM2-1.2B shape: 64 rows
// 38.95 k against 37.63 k tok/s with the kernel for 17 to 64 rows, 32 rows 26.0 k against 25.1 k;
// the LFM2-350M serving workload 35.1 k against 34.2 k generated tok/s.
#define KAPPAI_ROWS32_MIN_ROWS 24
#define KAPPAI_ROWS32_MAX_ROWS 128
// K of a block of that kernel comes in runs of this many
#define KAPPAI_ROWS32_RUN 256
