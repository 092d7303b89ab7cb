// Split-KV decode attention for callers that cannot allocate.
//
// This entry point has no counterpart in the reference.  It exists for callers that cannot call
// hipMalloc: code under HIP graph capture, tight serving loops, and harnesses that forbid allocation.
// It is arle_attn_paged_mfma restricted to steps whose every segment fits one row tile of 16 (single
// decoded tokens above all), with the split-KV partial results (o, and the pair m, l of every
// (token, q head, split)) kept in a fixed array in device memory of this library instead of a workspace
// that the caller brings.  Inputs and outputs are still the caller's.
//
// Limits: segments * ws_rows * nq * splits * D <= kAttnStaticOFloats and
// segments * ws_rows * nq * splits * 2 <= kAttnStaticMlFloats (ws_rows = arle_attn_ws_rows(max_qlen, nq, nkv));
// beyond them the call returns hipErrorInvalidValue and arle_attn_decode_static_error() says which
// size was too large.  The array takes (kAttnStaticOFloats + kAttnStaticMlFloats) * 4 bytes, 9 MiB, on
// every GPU this library runs on, until the process ends.
//
// Every call on a GPU shares that GPU's array, which keeps the last call's contents.  Nothing in it has to
// start at zero: each (token, q head, split) entry that the merge reads is written by the launch before it,
// in the same call.  Calls that overlap on one GPU (two streams, two threads) race on the array: run them
// on one stream, or one after the other.
//
// The call allocates nothing: no hipMalloc, hipFree or allocating library routine.  On its first call on a
// device it looks up that device's address of the array (hipGetSymbolAddress) and keeps it.
#pragma once

constexpr long long kAttnStaticOFloats = 2LL << 20;    // 8 MiB of partial outputs
constexpr long long kAttnStaticMlFloats = 256LL << 10;  // 1 MiB of (max, sum) pairs

extern "C" int arle_attn_decode_static(const void* q, long long q_stride, void* out, long long o_stride,
                                       const void* k_pages, const void* v_pages, const int* block_table,
                                       int table_stride, const int* seg_row0, const int* seg_slot,
                                       const int* seg_start, int segments, int max_qlen, int nq, int nkv, int D,
                                       int page_size, float scale, int window, int splits, void* stream);

// The reason of this thread's last refusal by arle_attn_decode_static ("" if there was none).
extern "C" const char* arle_attn_decode_static_error();
