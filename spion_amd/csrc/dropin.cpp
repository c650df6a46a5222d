// Drop-in libraries: re-export one family of libspion_hip.so under the un-prefixed names the
// reference's ctypes loaders bind (models/attention.py:141-191: init, attn_forward, attn_backward,
// destroy).  Built four times, once per SPION_DROPIN value:
//   1 -> attn.so            (models/attn.cu:265-280)
//   2 -> attn_mask.so       (models/attn_mask.cu:280-298)
//   3 -> block_attn.so      (models/block_attn.cu:547-568)
//   4 -> block_attn_mask.so (models/block_attn_mask.cu:655-674)
#include "../../include/spion_hip.h"

#ifndef SPION_DROPIN
#error "define SPION_DROPIN to 1..4"
#endif

#define EXPORT extern "C" __attribute__((visibility("default")))

#if SPION_DROPIN == 1
EXPORT void* init(int emb_dim, int seq_len, int num_batches) { return spion_dense_init(emb_dim, seq_len, num_batches); }
EXPORT void attn_forward(void* h, float* Qt, float* K, float* Vt, float* Attn, float* Out) {
    spion_dense_attn_forward(h, Qt, K, Vt, Attn, Out);
}
EXPORT void attn_backward(void* h, float* Qt, float* Kt, float* V, float* P, float* dOt, float* dP, float* dScale,
                          float* dS, float* dQ, float* dK, float* dV) {
    spion_dense_attn_backward(h, Qt, Kt, V, P, dOt, dP, dScale, dS, dQ, dK, dV);
}
EXPORT void destroy(void* h) { spion_dense_destroy(h); }

#elif SPION_DROPIN == 2
EXPORT void* init(int emb_dim, int seq_len, int num_batches) {
    return spion_densemask_init(emb_dim, seq_len, num_batches);
}
EXPORT void attn_forward(void* h, float* Qt, float* K, float* Vt, float* Mask, float* Attn, float* Out) {
    spion_densemask_attn_forward(h, Qt, K, Vt, Mask, Attn, Out);
}
EXPORT void attn_backward(void* h, float* Qt, float* Kt, float* V, float* P, float* dOt, float* dP, float* dScale,
                          float* dS, float* dQ, float* dK, float* dV) {
    spion_densemask_attn_backward(h, Qt, Kt, V, P, dOt, dP, dScale, dS, dQ, dK, dV);
}
EXPORT void destroy(void* h) { spion_densemask_destroy(h); }

#elif SPION_DROPIN == 3
EXPORT void* init(int emb_dim, int seq_len, int num_batches, int block_size) {
    return spion_block_init(emb_dim, seq_len, num_batches, block_size);
}
EXPORT void attn_forward(void* h, float* Q, float* Kt, float* V, float* Attn, float* Out, int* Offsets, int* Columns,
                         int* SumMat, int nnz) {
    spion_block_attn_forward(h, Q, Kt, V, Attn, Out, Offsets, Columns, SumMat, nnz);
}
EXPORT void attn_backward(void* h, float* Q, float* K, float* Vt, float* P, float* dO, float* dP, float* dS, float* dQ,
                          float* dK, float* dV, int* Offsets, int* Columns, int* SumMat, int nnz) {
    spion_block_attn_backward(h, Q, K, Vt, P, dO, dP, dS, dQ, dK, dV, Offsets, Columns, SumMat, nnz);
}
EXPORT void destroy(void* h) { spion_block_destroy(h); }

#elif SPION_DROPIN == 4
EXPORT void* init(int emb_dim, int seq_len, int num_batches, int block_size) {
    return spion_blockmask_init(emb_dim, seq_len, num_batches, block_size);
}
EXPORT void attn_forward(void* h, float* Q, float* Kt, float* V, float* Mask, float* Attn, float* Out, int* Offsets,
                         int* Columns, int* SumMat, int nnz) {
    spion_blockmask_attn_forward(h, Q, Kt, V, Mask, Attn, Out, Offsets, Columns, SumMat, nnz);
}
EXPORT void attn_backward(void* h, float* Q, float* K, float* Vt, float* P, float* dO, float* dP, float* dS, float* dQ,
                          float* dK, float* dV, int* Offsets, int* Columns, int* SumMat, int nnz) {
    spion_blockmask_attn_backward(h, Q, K, Vt, P, dO, dP, dS, dQ, dK, dV, Offsets, Columns, SumMat, nnz);
}
EXPORT void destroy(void* h) { spion_blockmask_destroy(h); }
#else
#error "SPION_DROPIN must be 1..4"
#endif
