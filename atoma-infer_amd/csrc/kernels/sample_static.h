// Sampling for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc.  This entry point has no counterpart in the reference (which samples on the
// host, backends/vllm/src/llm_service.rs:346-372); it is atoma_sample without the workspace argument.
//
// atoma_sample needs rows * vocab floats of device memory beside its inputs and outputs (the rows' weights
// exp((l - max) / T), walked several times by the top-k / top-p search and the draw).  Here that memory is an array
// inside the library's code object, of ATOMA_SAMPLE_STATIC_MAX_FLOATS floats (8 MiB), which every device the library
// runs on holds until the process ends.  The call allocates and frees nothing, neither through HIP nor through torch.
//
//   rc = atoma_sample_static(logits, ld, rows, vocab, temperature, top_k, top_p, uniform, out_token, out_logit, stream)
//
// takes the same inputs and writes the same outputs as atoma_sample (same kernel, same bits).
//   * rows * vocab > ATOMA_SAMPLE_STATIC_MAX_FLOATS returns ATOMA_ERR_TOO_LARGE (-4) and launches nothing.
//   * The array's device address is looked up once per device, at the first call on that device with that device
//     current, or ahead of time by atoma_sample_static_init() (a caller that is going to capture calls it first).
//   * All calls on one device share the array and it keeps the last call's contents: calls that overlap in time on
//     one device (different streams or threads) race with each other.  Calls in one stream do not.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define ATOMA_SAMPLE_STATIC_MAX_FLOATS (1u << 21)
#define ATOMA_ERR_TOO_LARGE (-4)

extern "C" int atoma_sample_static_init(void);
extern "C" int atoma_sample_static(const float* logits, int ld, int n_rows, int vocab, const float* temperature,
                                   const int32_t* top_k, const float* top_p, const float* uniform,
                                   int32_t* out_token, float* out_logit, hipStream_t stream);
