/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's fused-embedding semantics.
 * Nothing in the product (recflex_amd/, bench.py's measured path) may call this; only tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline leg do, as the checker.
 *
 * What it restates (paths relative to the reference repository):
 *  - oracle_pool_feature / oracle_pool_fused: the definition of the fused op used by the
 *    reference's only numerical check, examples/test.py:68-86: for every feature and sample,
 *    output[sample, dim_offset : dim_offset + D] = sum over the sample's indices of the table
 *    row (F.embedding(indices, table).sum(0)); empty line -> zeros; features concatenated along
 *    dim 1 in feature order (column offsets = prefix sums of the dims,
 *    RecFlex/code_emitter/codegen.py:227-231,289-292).  Summation is sequential, left to
 *    right, in fp32 -- the order of the reference's warp-per-sample kernel
 *    (examples/csrc/include/warp_per_sample_kernel.cuh:48-60) and, bit for bit, of torch's CPU
 *    embedding_bag(mode="sum") on fp32.
 *  - fp16 and int8 tables do not exist in the reference.  Their numerics are DEFINED here as
 *    "decode the row to fp32, then the same fp32 sum": fp16 -> exact widening; int8 row =
 *    D unsigned codes + fp16 scale + fp16 bias, value = (float)code * scale + bias (one fp32
 *    multiply, one fp32 add, no fma).  Parity for these two element types is therefore
 *    "parity unpinned" with respect to the reference (nothing there to compare with); the
 *    decode itself is pinned by closed-form tests in tests/test_oracle.py.
 *  - oracle_parse_lines: the digit / non-digit splitter of
 *    examples/csrc/warp_per_sample_preprocess.cu:9-38 and its offsets (exclusive prefix sum of
 *    the bag lengths, [B+1]).
 *
 * oracle/_ref: not built.  The reference's own path is CUDA (nvcc, CUB, a torch CUDA
 * extension: RecFlex/sched_basic_csrc/CMakeLists.txt, examples/csrc/CMakeLists.txt) and even its
 * host parsers include CUB headers; none of that exists in this image, so it is unbuildable
 * here.
 */
#include <stdint.h>
#include <string.h>

#define ORACLE_F32 0
#define ORACLE_F16 1
#define ORACLE_I8 2

static float half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int shift = 0;
      while (!(man & 0x400u)) { man <<= 1; ++shift; }
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

float oracle_half_to_float(uint16_t h) { return half_to_float(h); }

/* One feature: out[b * out_stride + col_off + d] for b in [0, batch), d in [0, dim).
 * table: rows of row_stride bytes.  Returns 0, or -1 on a bad dtype, -2 on an index outside
 * [0, rows). */
int oracle_pool_feature(const void *table, int dtype, int64_t rows, int dim, int row_stride,
                        const int32_t *indices, const int32_t *offsets, int batch, float *out,
                        int64_t out_stride, int col_off) {
  const unsigned char *base = (const unsigned char *)table;
  for (int b = 0; b < batch; ++b) {
    float *dst = out + (int64_t)b * out_stride + col_off;
    for (int d = 0; d < dim; ++d) dst[d] = 0.0f;
    for (int32_t p = offsets[b]; p < offsets[b + 1]; ++p) {
      const int64_t r = indices[p];
      if (r < 0 || r >= rows) return -2;
      const unsigned char *row = base + r * (int64_t)row_stride;
      if (dtype == ORACLE_F32) {
        const float *w = (const float *)row;
        for (int d = 0; d < dim; ++d) dst[d] += w[d];
      } else if (dtype == ORACLE_F16) {
        const uint16_t *w = (const uint16_t *)row;
        for (int d = 0; d < dim; ++d) dst[d] += half_to_float(w[d]);
      } else if (dtype == ORACLE_I8) {
        uint16_t sb[2];
        memcpy(sb, row + dim, 4);
        const float scale = half_to_float(sb[0]);
        const float bias = half_to_float(sb[1]);
        for (int d = 0; d < dim; ++d) {
          volatile float prod = (float)row[d] * scale; /* keep mul and add separate */
          dst[d] += prod + bias;
        }
      } else {
        return -1;
      }
    }
  }
  return 0;
}

/* All features, concatenated along dim 1 in feature order. */
int oracle_pool_fused(int num_features, const void *const *tables, const int32_t *dtypes,
                      const int64_t *rows, const int32_t *dims, const int32_t *row_strides,
                      const int32_t *const *indices, const int32_t *const *offsets, int batch,
                      float *out) {
  int64_t dim_sum = 0;
  for (int f = 0; f < num_features; ++f) dim_sum += dims[f];
  int col_off = 0;
  for (int f = 0; f < num_features; ++f) {
    const int rc = oracle_pool_feature(tables[f], dtypes[f], rows[f], dims[f], row_strides[f],
                                       indices[f], offsets[f], batch, out, dim_sum, col_off);
    if (rc) return rc;
    col_off += dims[f];
  }
  return 0;
}

/* Lines of one feature ('\n' separated, no trailing '\n' needed) -> indices, offsets[num_lines+1].
 * Returns the number of indices, or -1 if the text does not hold exactly num_lines lines (one
 * final '\n' is tolerated) or capacity is too small. */
int64_t oracle_parse_lines(const char *text, int64_t len, int num_lines, int32_t *indices,
                           int64_t capacity, int32_t *offsets) {
  int64_t n = 0, pos = 0;
  offsets[0] = 0;
  for (int line = 0; line < num_lines; ++line) {
    if (pos > len) return -1; /* the text holds fewer lines */
    int64_t end = pos;
    while (end < len && text[end] != '\n') ++end;
    /* the reference's loop over one std::string (warp_per_sample_preprocess.cu:14-29) */
    int32_t index = 0;
    for (int64_t i = pos; i < end; ++i) {
      const char ch = text[i];
      if (ch < '0' || ch > '9') {
        if (n >= capacity) return -1;
        indices[n++] = index;
        index = 0;
      } else {
        index = index * 10 + (ch - '0');
      }
    }
    if (end > pos) {
      if (n >= capacity) return -1;
      indices[n++] = index;
    }
    offsets[line + 1] = (int32_t)n;
    pos = end + 1;
  }
  if (pos < len) return -1; /* the text holds more lines */
  return n;
}
