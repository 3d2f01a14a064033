// Sampling for callers that cannot allocate device memory: code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc.  This entry point has no
// counterpart in the reference; it is here for those callers only.
//
// ts_sample_static does what ts_sample does (row r: greedy if temperature[r] <= 1e-10,
// else a draw from softmax(logits[r] / T) with noise keyed by keys[r]), but the winners
// of the vocabulary slices, which ts_sample takes as the caller's part_v / part_i
// workspace, lie in a file-scope device array of the library.  It allocates nothing, on
// the host or the device.
//
// Limit: rows * ts_pick_slices(vocab) <= ts_sample_static_capacity() (65,536 slice
// winners, 512 KiB of device memory that every GPU the library runs on holds until the
// process ends); more is refused with an error, never served from elsewhere.
//
// Every call on one GPU uses that GPU's one array, so two calls that overlap on one GPU
// (different streams, or different threads) race: the caller orders them.  Nothing in
// the array has to start at zero: the first kernel writes every entry the second reads,
// and entries of an earlier, larger call beyond that are never read.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" int ts_sample_static_capacity();
extern "C" int ts_sample_static(const float* logits, const float* temperature,
                                const uint64_t* keys, int* out, int rows, int vocab,
                                hipStream_t stream);
