// ABI version, error strings and the host-side integer chunk bookkeeping.
#include "fla_common.h"

extern "C" int fla_abi_version(void) { return FLA_ABI_VERSION; }

extern "C" const char* fla_error_string(int code) {
  switch (code) {
    case FLA_OK: return "success";
    case FLA_E_INVALID: return "fla_hip: invalid argument (null pointer, negative size or inconsistent shapes)";
    case FLA_E_UNSUPPORTED: return "fla_hip: shape, dtype or chunk size not supported by the gfx950 kernels";
    case FLA_E_ALIGNMENT: return "fla_hip: pointer or row pitch not aligned for vector access";
    case FLA_E_SCRATCH: return "fla_hip: input larger than the static scratch buffer of the allocation-free entry point";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "fla_hip: unknown error code";
}

// One row (sequence, chunk-in-sequence) per chunk, sequences in order, and the
// exclusive prefix sum of per-sequence chunk counts.  Same result as the
// reference's host construction (fla/ops/gla/chunk.py:1323-1330;
// fla/ops/common/chunk_h.py:274-279), without a device round trip.
extern "C" int64_t fla_count_chunks(const int64_t* offsets, int64_t n_seqs, int64_t chunk_size) {
  if (!offsets || n_seqs < 0 || chunk_size <= 0) return FLA_E_INVALID;
  int64_t total = 0;
  for (int64_t n = 0; n < n_seqs; ++n) {
    int64_t len = offsets[n + 1] - offsets[n];
    if (len < 0) return FLA_E_INVALID;
    total += fla_cdiv(len, chunk_size);
  }
  return total;
}

extern "C" int fla_prepare_chunk_indices(const int64_t* offsets, int64_t n_seqs, int64_t chunk_size,
                                         int64_t* indices_out, int64_t* chunk_offsets_out) {
  if (!offsets || n_seqs < 0 || chunk_size <= 0) return FLA_E_INVALID;
  int64_t row = 0;
  for (int64_t n = 0; n < n_seqs; ++n) {
    int64_t len = offsets[n + 1] - offsets[n];
    if (len < 0) return FLA_E_INVALID;
    if (chunk_offsets_out) chunk_offsets_out[n] = row;
    int64_t nc = fla_cdiv(len, chunk_size);
    for (int64_t c = 0; c < nc; ++c, ++row) {
      if (indices_out) {
        indices_out[2 * row] = n;
        indices_out[2 * row + 1] = c;
      }
    }
  }
  if (chunk_offsets_out) chunk_offsets_out[n_seqs] = row;
  return FLA_OK;
}
