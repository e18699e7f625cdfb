// CPU side of the fused-embedding path: dataset text -> indices / offsets -> packed buffer.
// Exports the recom_host_* entry points declared in include/recflex_hip.h.
//
// Reference behaviour reproduced: the digit/non-digit line splitter of
// examples/csrc/warp_per_sample_preprocess.cu:9-38 (identical copies in
// one_block_multi_sample_preprocess.cu and multi_block_per_sample_preprocess.cu), and the
// 128-byte padding of every vector in the argument buffer
// (RecFlex/code_emitter/codegen.py:149-160, RecFlex/sched_basic_csrc/include/utils.cuh:60-68).
#include "recflex_hip.h"

#include <cstring>

extern "C" {

int64_t recom_host_max_indices(int64_t text_len) {
  // every index needs at least one byte and indices are separated by at least one byte;
  // "," alone holds two (empty) indices
  return text_len < 0 ? 0 : text_len + 1;
}

int64_t recom_host_alignmem(int64_t nbytes) { return (nbytes + 127) / 128 * 128; }

int64_t recom_host_packed_size(int32_t batch, int64_t num_indices) {
  return recom_host_alignmem((static_cast<int64_t>(batch) + 1) * 4) +
         recom_host_alignmem(num_indices * 4);
}

int recom_host_parse_lines(const char *text, int64_t text_len, int32_t num_lines,
                           int32_t *indices_out, int64_t indices_capacity,
                           int32_t *offsets_out, int64_t *num_indices_out) {
  if ((!text && text_len > 0) || text_len < 0 || num_lines < 0 || !offsets_out ||
      !num_indices_out || (!indices_out && indices_capacity > 0))
    return RECOM_HOST_EINVAL;

  int64_t n = 0;      // indices written
  int32_t line = 0;   // lines finished
  int64_t value = 0;
  bool line_nonempty = false;
  offsets_out[0] = 0;

  auto push = [&](int64_t v) -> int {
    if (v > INT32_MAX) return RECOM_HOST_ERANGE;
    if (n >= indices_capacity) return RECOM_HOST_ENOSPC;
    indices_out[n++] = static_cast<int32_t>(v);
    return 0;
  };
  auto end_line = [&]() -> int {
    if (line_nonempty) {
      if (int rc = push(value)) return rc;
    }
    if (line >= num_lines) return RECOM_HOST_ELINES;
    if (n > INT32_MAX) return RECOM_HOST_ERANGE;
    offsets_out[++line] = static_cast<int32_t>(n);
    value = 0;
    line_nonempty = false;
    return 0;
  };

  for (int64_t i = 0; i < text_len; ++i) {
    const char ch = text[i];
    if (ch == '\n') {
      if (int rc = end_line()) return rc;
    } else if (ch < '0' || ch > '9') {
      if (int rc = push(value)) return rc;
      value = 0;
      line_nonempty = true;
    } else {
      value = value * 10 + (ch - '0');
      if (value > INT32_MAX) return RECOM_HOST_ERANGE;
      line_nonempty = true;
    }
  }
  // last line without a terminating '\n' (also the empty last line of "a\n" + "")
  if (line < num_lines) {
    if (int rc = end_line()) return rc;
  } else if (line_nonempty) {
    return RECOM_HOST_ELINES;
  }
  if (line != num_lines) return RECOM_HOST_ELINES;
  *num_indices_out = n;
  return 0;
}

int recom_host_pack(int32_t num_features, int32_t batch, const int32_t *const *offsets,
                    const int32_t *const *indices, const int64_t *num_indices, void *dst,
                    int64_t dst_capacity, int64_t *byte_offsets_out) {
  if (num_features < 0 || batch < 0 || !byte_offsets_out ||
      (num_features > 0 && (!offsets || !indices || !num_indices || !dst)))
    return RECOM_HOST_EINVAL;
  char *out = static_cast<char *>(dst);
  int64_t pos = 0;
  byte_offsets_out[0] = 0;
  for (int32_t f = 0; f < num_features; ++f) {
    if (num_indices[f] < 0 || !offsets[f] || (num_indices[f] > 0 && !indices[f]))
      return RECOM_HOST_EINVAL;
    const int64_t off_bytes = (static_cast<int64_t>(batch) + 1) * 4;
    const int64_t idx_bytes = num_indices[f] * 4;
    const int64_t off_pad = recom_host_alignmem(off_bytes);
    const int64_t idx_pad = recom_host_alignmem(idx_bytes);
    if (pos + off_pad + idx_pad > dst_capacity) return RECOM_HOST_ENOSPC;
    std::memcpy(out + pos, offsets[f], off_bytes);
    std::memset(out + pos + off_bytes, 0, off_pad - off_bytes);
    pos += off_pad;
    if (idx_bytes) std::memcpy(out + pos, indices[f], idx_bytes);
    std::memset(out + pos + idx_bytes, 0, idx_pad - idx_bytes);
    pos += idx_pad;
    byte_offsets_out[f + 1] = pos;
  }
  return 0;
}

} // extern "C"
