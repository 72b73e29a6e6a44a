/* Flat C API of the host-side front-end (libug_host.so).  Handles are opaque `void*`:
 *   device    -> shared ug::Device        slice -> ug::Slice          func -> shared ug::Func
 *   lb        -> ug::LazyBuffer           ssa   -> ug::ssa::Kernel    schedule / compiled / cache
 * A device created by another library (e.g. the CPU oracle used by the tests) plugs into every
 * function here, because all of them go through the abstract ug::Device. */
#ifndef UGH_CAPI_H_
#define UGH_CAPI_H_
#include <stddef.h>
#include <stdint.h>

#include "ughip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* custom-op callback: slices are `slice` handles, inputs first, destination last. */
typedef int (*ugh_custom_fn)(void* user, void** slices, size_t n);

typedef struct ugh_llama_config {
  size_t hidden_size, intermediate_size, max_position_embeddings;
  size_t num_attention_heads, num_key_value_heads, num_hidden_layers;
  double rms_norm_eps;
  int rope_interleaved;
  float rope_theta;
  size_t vocab_size;
} ugh_llama_config;

const char* ugh_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
