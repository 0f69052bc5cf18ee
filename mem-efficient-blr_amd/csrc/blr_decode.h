// Two-stage BLAST decode kernel (blr_decode.hip), called from the streaming engine's BLAST entry.
#pragma once
#include "blr_common.h"

namespace blr {

// Bytes of the fixed-place workspace block that holds the tagged values exchanged by workgroups.
size_t decode2_region_bytes();
// Bytes of the fixed-place workspace block behind it that the multi-launch paths use as ordinary scratch (y, z, re-laid S).
// It is a block of its own so that no plain value is ever left where a single-launch kernel looks for a tagged one.
size_t decode2_plain_bytes();
// Whether the call can be served by the two-stage decode kernel at all (layout, dtype, M).
bool decode2_applicable(const StreamBlastArgs& a);
// Returns BLR_OK, a negative blr_status, or 1 when the shape does not fit the kernel's tiling
// (the caller then uses the phase engine).
int decode2_blast_launch(const StreamBlastArgs& a, void* region, void* plain, unsigned* epoch_word, unsigned* arrive_word,
                         unsigned* err_word, hipStream_t st);

// The same call on the one-workgroup-per-compute-unit kernel (blr_decode3.hip; up to four token rows).  Returns BLR_OK, a
// negative blr_status, or 1 when the call is not for it (decode2_blast_launch then serves it itself).
int decode3_blast_launch(const StreamBlastArgs& a, void* region, unsigned* epoch_word, unsigned* arrive_word,
                         unsigned* err_word, hipStream_t st);

// The same call as two launches - stage 1, then mix + stage 2 - with ordinary memory between them (blr_decode_pair.hip; up
// to four token rows, U (b, r, q), S with the rank contiguous).  region: scratch for y as T.  Same return convention.
int decode_pair_launch(const StreamBlastArgs& a, void* region, size_t region_bytes, hipStream_t st);

// The same call as three launches - y = x V and out = z U on the matrix cores with the rank-space mix between them
// (blr_decode_rows.hip; up to 128 token rows in tiles of 16, two-byte weights or codes).  region: scratch for y and z as T.  Same
// return convention.
int decode_rows_launch(const StreamBlastArgs& a, void* region, size_t region_bytes, hipStream_t st);

// Dense layer out = x W (W (in_f, out_f) row-major) at 17..128 token rows with the same product kernel: the reduction is cut
// into equal slices of at most 1024 rows of W (so that the weights of a chunk stay in registers over the tiles of 16 token
// rows), every slice leaves its partial product as T in `ws`, and one more launch adds the slices in fp32.  dense_rows_bytes:
// bytes of the partial products, 0 when the shape is not for this path; the launch returns 1 then.
size_t dense_rows_bytes(int M, int in_f, int out_f, int dtype);
int dense_rows_launch(const void* x, int64_t ldx, const void* W, void* out, int64_t ldo, int M, int in_f, int out_f, int dtype,
                      void* ws, size_t ws_bytes, hipStream_t st);

// Dense layer out = x W (W (K, N)) at up to 16 rows: slabs of W on the matrix cores, fp32 partial sums of the k-slices in `part`
// (room for max_slices * M * N floats) added by a second launch.  Returns BLR_OK, a negative blr_status, or 1 when the
// call is not for this kernel.
int dense_slab_launch(const void* x, int64_t ldx, const void* W, void* out, int64_t ldo, int M, int K, int N, int dtype,
                      float* part, int max_slices, hipStream_t st);

// The same kernel for a batch of products C[bt] = A[bt] B[bt] with B (K, N) row-major (row stride ldb, batch strides in elements).
// Without a partial-sum area (part null) the reduction is not cut and K is limited to one slab (1024 rows).
int slab_gemm_launch(const void* A, int64_t lda, int64_t sA, const void* B, int64_t ldb, int64_t sB, void* C, int64_t ldc, int64_t sC,
                     int M, int N, int K, int batch, int dtype, float* part, int max_slices, hipStream_t st);

}  // namespace blr
