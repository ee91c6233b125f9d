// An entry point of the kernel library that allocates nothing.
//
// It has no counterpart in the reference. It is for callers that cannot allocate device memory: code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc. jllm_decode_attention_bf16 takes its
// scratch (the partial sums of the key splits) from the caller; this variant runs the same kernels with the
// scratch in an array that is part of the library's device image, so nothing is allocated or freed by the call,
// neither by the HIP runtime nor by a library.
//
// Limits and rules:
//  * the scratch holds JLLM_NO_ALLOC_SCRATCH_FLOATS floats (16 MiB), which every GPU the library runs on keeps
//    until the process ends; a call needs n_rows * H * (max_pos / split + 1) * (hd + 2) floats and is refused with
//    an error (return -1, text in jllm_last_error) when that is more;
//  * every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two threads)
//    race; calls on one stream follow each other and are safe;
//  * nothing in the scratch has to start at zero: the first kernel writes every entry that the second one reads,
//    so what the call before left there is never seen;
//  * the array's device address is looked up once per GPU, on the first call with that GPU current (that call
//    must not be inside a graph capture).
#pragma once
#include <hip/hip_runtime.h>

#define JLLM_NO_ALLOC_SCRATCH_FLOATS (4u << 20)

// As jllm_decode_attention_bf16 (same arguments, same kernels, same results bit for bit), without part_acc,
// part_ml and max_splits. Returns 0 when it ran, 1 when the kernels do not take the shape, -1 on errors.
extern "C" int jllm_decode_attention_bf16_no_alloc(const void* q, int ldq, void* out, int ldo, const void* kcache,
                                                   const void* vcache, const int* block_table, int max_blocks,
                                                   const int* row_req, const int* positions, int n_rows, int H,
                                                   int Hkv, int hd, int page_size, int window, float scale,
                                                   int max_pos, int split, hipStream_t stream);
