// Peregrine's int8 wire record for a quantised tensor (serial::write_quantized_tensor /
// read_quantized_tensor, reference src/serial.rs:124-222):
//   [name_len u32][name bytes][dtype u8 = 1][ndim u32 = 2][rows u32][cols u32]
//   [rows*cols i8, row-major [rows, cols]][cols f32 scales]          all little-endian.
// Host code; pg_qtensor_from_record hands the payload to pg_qtensor_upload, whose device
// layout is the "pre-transpose for GEMM" the reference's reader does on the host
// (src/serial.rs:202-208).
#include "pg_internal.h"

namespace {
constexpr size_t FIXED = 4 + 1 + 4 + 4 + 4;  // name_len, dtype, ndim, rows, cols

void put_u32(uint8_t *&p, uint32_t v) { memcpy(p, &v, 4); p += 4; }
}  // namespace

PG_API pg_status pg_quantized_record_size(size_t name_len, size_t rows, size_t cols, size_t *bytes) {
    PG_CHECK_ARG(bytes != nullptr, "pg_quantized_record_size: null output");
    PG_CHECK_ARG(name_len <= 0xFFFFFFFFull && rows <= 0xFFFFFFFFull && cols <= 0xFFFFFFFFull,
                 "pg_quantized_record_size: a field does not fit the format's u32");
    *bytes = FIXED + name_len + rows * cols + cols * sizeof(float);
    return PG_OK;
}

PG_API pg_status pg_write_quantized_tensor(void *buf, size_t cap, const char *name, size_t name_len, const int8_t *q,
                                           const float *scales, size_t rows, size_t cols, size_t *written) {
    size_t need = 0;
    PG_TRY(pg_quantized_record_size(name_len, rows, cols, &need));
    PG_CHECK_ARG(buf != nullptr && cap >= need, "pg_write_quantized_tensor: buffer holds %zu of %zu bytes", cap, need);
    PG_CHECK_ARG((name || name_len == 0) && (q || rows * cols == 0) && (scales || cols == 0),
                 "pg_write_quantized_tensor: null pointer");
    uint8_t *p = static_cast<uint8_t *>(buf);
    put_u32(p, (uint32_t)name_len);
    memcpy(p, name, name_len); p += name_len;
    *p++ = 1;  // dtype tag: i8 quantised
    put_u32(p, 2);
    put_u32(p, (uint32_t)rows);
    put_u32(p, (uint32_t)cols);
    memcpy(p, q, rows * cols); p += rows * cols;
    memcpy(p, scales, cols * sizeof(float));
    if (written) *written = need;
    return PG_OK;
}

PG_API pg_status pg_read_quantized_tensor(const void *buf, size_t len, const char **name, size_t *name_len, size_t *rows,
                                          size_t *cols, const int8_t **q, const void **scales, size_t *consumed) {
    PG_CHECK_ARG(buf != nullptr || len == 0, "pg_read_quantized_tensor: null buffer");
    const uint8_t *p = static_cast<const uint8_t *>(buf);
    auto short_read = [&]() { return pg_fail(PG_EINVAL, "pg_read_quantized_tensor: record is truncated (%zu bytes)", len); };
    if (len < 4) return short_read();
    uint32_t nl, ndim, r, c;
    memcpy(&nl, p, 4);
    if (len - 4 < (size_t)nl || len - 4 - nl < FIXED - 4) return short_read();
    const uint8_t *h = p + 4 + nl;
    PG_CHECK_ARG(h[0] == 1, "expected dtype=1 (i8) for quantized tensor, got %u", (unsigned)h[0]);  // src/serial.rs:176
    memcpy(&ndim, h + 1, 4);
    PG_CHECK_ARG(ndim == 2, "quantized tensors must be 2D, got ndim=%u", ndim);  // src/serial.rs:181
    memcpy(&r, h + 5, 4);
    memcpy(&c, h + 9, 4);
    const size_t head = 4 + (size_t)nl + (FIXED - 4), body = (size_t)r * c + (size_t)c * sizeof(float);
    if (len - head < body) return short_read();
    if (name) *name = reinterpret_cast<const char *>(p + 4);
    if (name_len) *name_len = nl;
    if (rows) *rows = r;
    if (cols) *cols = c;
    if (q) *q = reinterpret_cast<const int8_t *>(p + head);
    if (scales) *scales = p + head + (size_t)r * c;  // not necessarily 4-byte aligned
    if (consumed) *consumed = head + body;
    return PG_OK;
}

PG_API pg_status pg_qtensor_from_record(pg_ctx *ctx, const void *buf, size_t len, pg_qtensor **out, size_t *consumed) {
    PG_CHECK_ARG(out != nullptr, "pg_qtensor_from_record: out is null");
    *out = nullptr;
    size_t rows = 0, cols = 0;
    const int8_t *q = nullptr;
    const void *sc = nullptr;
    PG_TRY(pg_read_quantized_tensor(buf, len, nullptr, nullptr, &rows, &cols, &q, &sc, consumed));
    PG_CHECK_ARG(rows > 0 && cols > 0, "pg_qtensor_from_record: empty tensor");
    std::vector<float> scales(cols);  // aligned copy
    memcpy(scales.data(), sc, cols * sizeof(float));
    return pg_qtensor_upload(ctx, q, scales.data(), rows, cols, out);
}
