// C ABI, part: repacked weight handles (one-time repack at upload, one or two copies, fusing along N) and their
// byte blob for an on-disk cache.
#include "twm_api_impl.h"

using namespace twm;

extern "C" {

/* ---- repacked weights ----------------------------------------------------------------------- */

extern "C++" twm_weight *weight_alloc(twm_ctx *ctx, uint32_t k, uint32_t n)
{
    twm_weight *w = new (std::nothrow) twm_weight();
    if (!w) { api_fail(TWM_MEMORY_ERROR, "twm_weight: out of host memory"); return nullptr; }
    w->ctx = ctx;
    w->k = k;
    w->n = n;
    w->groups = k / 32;
    uint32_t n_pad = ((n + kNPadTo - 1) / kNPadTo) * kNPadTo;
    w->n_tiles = n_pad / kTileN;
    w->k_chunks = (w->groups + kChunkGroups - 1) / kChunkGroups;
    size_t tiles = (size_t)w->n_tiles * w->k_chunks;
    w->copy_bytes = tiles * (1024 + 128);  // nibbles + scales: the same in either order
    w->bytes = 0;
    w->qw = w->sc = w->cq = nullptr;
    w->paired = false;
    memset(w->tuned, 0, sizeof w->tuned);
    return w;
}

// device memory for the copies in `mask` that the handle does not hold yet (contents undefined)
extern "C++" int weight_alloc_copies(twm_weight *w, int mask, const char *who)
{
    if (w->copy_bytes == 0) return TWM_OK;
    if ((mask & kCopyTile) && !w->qw) {
        hipError_t e = hipMalloc(&w->qw, w->copy_bytes);
        if (e != hipSuccess) { w->qw = nullptr; return api_fail(TWM_MEMORY_ERROR, "%s: hipMalloc(%zu): %s", who, w->copy_bytes, hipGetErrorString(e)); }
        w->sc = (char *)w->qw + (size_t)w->n_tiles * w->k_chunks * 1024;
        w->bytes += w->copy_bytes;
    }
    if ((mask & kCopyCol) && !w->cq) {
        hipError_t e = hipMalloc(&w->cq, w->copy_bytes);
        if (e != hipSuccess) { w->cq = nullptr; return api_fail(TWM_MEMORY_ERROR, "%s: hipMalloc(%zu): %s", who, w->copy_bytes, hipGetErrorString(e)); }
        w->bytes += w->copy_bytes;
    }
    return TWM_OK;
}

extern "C++" void weight_release(twm_weight *w)
{
    if (w->qw) (void)hipFree(w->qw);
    if (w->cq) (void)hipFree(w->cq);
    delete w;
}


// Makes sure the handle holds the copies in `mask`, building a missing one from the other on the context's stream.
// Allocates, so not inside a graph capture: a caller that captures its launches asks for the copies before
// (twm_weight_ensure, or option "weight_copies" when the handle is made).
extern "C++" int weight_ensure(twm_ctx *ctx, const twm_weight *cw, int mask, const char *who)
{
    twm_weight *w = const_cast<twm_weight *>(cw);  // (the handle is the library's own object; callers see it opaque)
    const int have = copies_of(w), missing = mask & ~have;
    if (!missing || w->copy_bytes == 0) return TWM_OK;
    if (ctx->capturing)
        return api_fail(TWM_UNSUPPORTED_OP, "%s: this call needs the weight's %s copy, which the handle does not hold, and building it "
                        "allocates: call twm_weight_ensure before the capture", who, (missing & kCopyTile) ? "16-column tile" : "column-lane");
    if (!have) return api_fail(TWM_INVALID_HANDLE, "%s: the weight holds no copy at all", who);
    if (int rc = weight_alloc_copies(w, missing, who)) return rc;
    hipError_t e = (missing & kCopyTile) ? launch_col_to_tile(ctx->stream, w->cq, w->n_tiles, w->k_chunks, w->qw, w->sc)
                                         : launch_tile_to_col(ctx->stream, w->qw, w->sc, w->n_tiles, w->k_chunks, w->cq);
    if (e != hipSuccess) return api_fail(TWM_DEVICE_ERROR, "%s: building the second weight copy: %s", who, hipGetErrorString(e));
    return TWM_OK;
}

int twm_weight_ensure(twm_ctx *ctx, twm_weight *w, int copies)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "twm_weight_ensure: null handle");
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "twm_weight_ensure: weight belongs to another context");
    if (copies < 1 || copies > 3) return api_fail(TWM_SHAPE_ERROR, "twm_weight_ensure: copies is 1 (16-column tiles), 2 (column-lane) or 3 (both)");
    return weight_ensure(ctx, w, copies, "twm_weight_ensure");
}

int twm_weight_drop(twm_ctx *ctx, twm_weight *w, int copies)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "twm_weight_drop: null handle");
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "twm_weight_drop: weight belongs to another context");
    if (ctx->capturing) return api_fail(TWM_UNSUPPORTED_OP, "twm_weight_drop: not allowed inside a graph capture");
    if (copies != kCopyTile && copies != kCopyCol) return api_fail(TWM_SHAPE_ERROR, "twm_weight_drop: copies is 1 (16-column tiles) or 2 (column-lane)");
    if (w->copy_bytes == 0 || !(copies_of(w) & copies)) return TWM_OK;
    if (copies_of(w) == copies) return api_fail(TWM_SHAPE_ERROR, "twm_weight_drop: that is the only copy the handle holds");
    HIP_TRY(hipStreamSynchronize(ctx->stream), TWM_DEVICE_ERROR, "twm_weight_drop: sync");
    if (copies == kCopyTile) { (void)hipFree(w->qw); w->qw = w->sc = nullptr; }
    else { (void)hipFree(w->cq); w->cq = nullptr; }
    w->bytes -= w->copy_bytes;
    return TWM_OK;
}

int twm_weight_copies(const twm_weight *w) { return w ? copies_of(w) : 0; }

// Option "tune_on_upload": a new plain weight handle gets its measured plans right away (twm_weight_tune over the row
// counts of decode, 1 = {1, 4, 8, 16, 32}, and with 2 also of prefill, {128, 512, 2048}).  A handle whose tuning fails is
// not returned: the caller asked for measured plans.
static twm_weight *tune_new_weight(twm_ctx *ctx, twm_weight *w)
{
    if (!w || !ctx->tune_on_upload || w->n == 0 || w->k == 0) return w;
    static const uint32_t ms[] = {1, 4, 8, 16, 32, 128, 512, 2048};
    if (twm_weight_tune(ctx, w, ms, ctx->tune_on_upload >= 2 ? 8u : 5u) != TWM_OK) {
        twm_weight_destroy(w);
        return nullptr;
    }
    return w;
}

static twm_weight *weight_from_device(twm_ctx *ctx, const uint8_t *packed_dev, const uint16_t *scales_dev, uint32_t k, uint32_t n);

twm_weight *twm_weight_from_device(twm_ctx *ctx, const uint8_t *packed_dev, const uint16_t *scales_dev, uint32_t k,
                                   uint32_t n)
{
    twm_weight *w = weight_from_device(ctx, packed_dev, scales_dev, k, n);
    return w ? tune_new_weight(ctx, w) : nullptr;
}

static twm_weight *weight_from_device(twm_ctx *ctx, const uint8_t *packed_dev, const uint16_t *scales_dev, uint32_t k, uint32_t n)
{
    if (!ctx) { api_fail(TWM_INVALID_HANDLE, "twm_weight_from_device: null context"); return nullptr; }
    if (ctx->capturing) { api_fail(TWM_UNSUPPORTED_OP, "twm_weight_from_device: not allowed inside a graph capture"); return nullptr; }
    if (check_kn("twm_weight_from_device", k, n)) return nullptr;
    if ((uint64_t)k * n != 0 && (!packed_dev || !scales_dev)) {
        api_fail(TWM_INVALID_HANDLE, "twm_weight_from_device: null pointer");
        return nullptr;
    }
    if (((uintptr_t)packed_dev & 3) != 0) { api_fail(TWM_SHAPE_ERROR, "twm_weight_from_device: packed must be 4-byte aligned"); return nullptr; }
    twm_weight *w = weight_alloc(ctx, k, n);
    if (!w) return nullptr;
    const int mask = ctx->weight_copies ? ctx->weight_copies : (kCopyTile | kCopyCol);
    if (weight_alloc_copies(w, mask, "twm_weight_from_device")) { weight_release(w); return nullptr; }
    if (w->copy_bytes) {
        hipError_t e = hipSuccess;
        if (w->qw) e = launch_repack(ctx->stream, packed_dev, scales_dev, k, n, w->qw, w->sc, w->n_tiles, w->k_chunks);
        if (e == hipSuccess && w->cq)
            e = launch_repack_col(ctx->stream, packed_dev, scales_dev, k, n, w->cq, w->n_tiles * kTileN, w->k_chunks);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) {
            api_fail(TWM_DEVICE_ERROR, "twm_weight_from_device: repack: %s", hipGetErrorString(e));
            weight_release(w);
            return nullptr;
        }
    }
    return w;
}

// Fusing along N on the repacked copies is block copying: the column-lane copy is tile-major (one contiguous run per
// input), the 16-column tile copy chunk-major (one 2-D copy per input: k_chunks rows of the input's tiles).
twm_weight *twm_weight_fuse_n(twm_ctx *ctx, const twm_weight *const *parts, uint32_t count)
{
    const char *who = "twm_weight_fuse_n";
    if (!ctx || !parts || count == 0) { api_fail(TWM_INVALID_HANDLE, "%s: null argument", who); return nullptr; }
    if (ctx->capturing) { api_fail(TWM_UNSUPPORTED_OP, "%s: not allowed inside a graph capture", who); return nullptr; }
    uint64_t total = 0;
    for (uint32_t i = 0; i < count; i++) {
        const twm_weight *p = parts[i];
        if (!p) { api_fail(TWM_INVALID_HANDLE, "%s: part %u is null", who, i); return nullptr; }
        if (p->ctx != ctx) { api_fail(TWM_INVALID_HANDLE, "%s: part %u belongs to another context", who, i); return nullptr; }
        if (p->k != parts[0]->k) { api_fail(TWM_SHAPE_ERROR, "%s: part %u has K = %u, part 0 has %u", who, i, p->k, parts[0]->k); return nullptr; }
        if (p->paired) { api_fail(TWM_UNSUPPORTED_OP, "%s: part %u is a paired gate/up weight", who, i); return nullptr; }
        if (i + 1 < count && p->n % kNPadTo != 0) {
            api_fail(TWM_SHAPE_ERROR, "%s: part %u has N = %u; every part but the last must be a multiple of %u columns "
                     "(fuse the arrays with twm_fuse_tw_marlin_n instead)", who, i, p->n, kNPadTo);
            return nullptr;
        }
        total += p->n;
    }
    if (total > 0xFFFFFFFFull) { api_fail(TWM_SHAPE_ERROR, "%s: fused N overflows u32", who); return nullptr; }
    if (check_kn(who, parts[0]->k, (uint32_t)total)) return nullptr;
    twm_weight *w = weight_alloc(ctx, parts[0]->k, (uint32_t)total);
    if (!w) return nullptr;
    const int mask = ctx->weight_copies ? ctx->weight_copies : (kCopyTile | kCopyCol);
    for (uint32_t i = 0; i < count; i++)
        if (weight_ensure(ctx, parts[i], mask, who)) { weight_release(w); return nullptr; }
    if (weight_alloc_copies(w, mask, who)) { weight_release(w); return nullptr; }
    hipError_t e = hipSuccess;
    uint32_t t16 = 0;  // 16-column tiles before this part
    for (uint32_t i = 0; i < count && e == hipSuccess && w->copy_bytes; i++) {
        const twm_weight *p = parts[i];
        if (p->n_tiles == 0) continue;
        if (w->cq)
            e = hipMemcpyAsync((char *)w->cq + (size_t)(t16 / 4) * w->k_chunks * kColBlockBytes, p->cq,
                               (size_t)(p->n_tiles / 4) * p->k_chunks * kColBlockBytes, hipMemcpyDeviceToDevice, ctx->stream);
        if (e == hipSuccess && w->qw)
            e = hipMemcpy2DAsync((char *)w->qw + (size_t)t16 * 1024, (size_t)w->n_tiles * 1024, p->qw, (size_t)p->n_tiles * 1024,
                                 (size_t)p->n_tiles * 1024, w->k_chunks, hipMemcpyDeviceToDevice, ctx->stream);
        if (e == hipSuccess && w->qw)
            e = hipMemcpy2DAsync((char *)w->sc + (size_t)t16 * 128, (size_t)w->n_tiles * 128, p->sc, (size_t)p->n_tiles * 128,
                                 (size_t)p->n_tiles * 128, w->k_chunks, hipMemcpyDeviceToDevice, ctx->stream);
        t16 += p->n_tiles;
    }
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        api_fail(TWM_DEVICE_ERROR, "%s: copy: %s", who, hipGetErrorString(e));
        weight_release(w);
        return nullptr;
    }
    return tune_new_weight(ctx, w);
}

twm_weight *twm_weight_upload(twm_ctx *ctx, const uint8_t *packed_host, const uint16_t *scales_host, uint32_t k,
                              uint32_t n)
{
    if (!ctx) { api_fail(TWM_INVALID_HANDLE, "twm_weight_upload: null context"); return nullptr; }
    if (ctx->capturing) { api_fail(TWM_UNSUPPORTED_OP, "twm_weight_upload: not allowed inside a graph capture"); return nullptr; }
    if (check_kn("twm_weight_upload", k, n)) return nullptr;
    size_t pbytes = (size_t)(k / 32) * n * 16, sbytes = (size_t)(k / 32) * n * 2;
    if (pbytes == 0) return weight_from_device(ctx, nullptr, nullptr, k, n);
    if (!packed_host || !scales_host) { api_fail(TWM_INVALID_HANDLE, "twm_weight_upload: null pointer"); return nullptr; }
    void *stage = nullptr;
    hipError_t e = hipMalloc(&stage, pbytes + sbytes);
    if (e != hipSuccess) { api_fail(TWM_MEMORY_ERROR, "twm_weight_upload: staging hipMalloc: %s", hipGetErrorString(e)); return nullptr; }
    uint8_t *p = (uint8_t *)stage;
    uint16_t *s = (uint16_t *)(p + pbytes);
    twm_weight *w = nullptr;
    if (twm_memcpy_h2d(ctx, p, packed_host, pbytes) == TWM_OK && twm_memcpy_h2d(ctx, s, scales_host, sbytes) == TWM_OK)
        w = weight_from_device(ctx, p, s, k, n);
    (void)hipFree(stage);
    return w ? tune_new_weight(ctx, w) : nullptr;
}

twm_weight *twm_weight_gate_up(twm_ctx *ctx, const uint8_t *gate_packed_dev, const uint16_t *gate_scales_dev,
                               const uint8_t *up_packed_dev, const uint16_t *up_scales_dev, uint32_t k, uint32_t ffn_dim)
{
    if (!ctx) { api_fail(TWM_INVALID_HANDLE, "twm_weight_gate_up: null context"); return nullptr; }
    if (ctx->capturing) { api_fail(TWM_UNSUPPORTED_OP, "twm_weight_gate_up: not allowed inside a graph capture"); return nullptr; }
    if (check_pair_args("twm_weight_gate_up", k, ffn_dim)) return nullptr;
    uint32_t n = ffn_dim * 2;
    size_t pbytes = (size_t)(k / 32) * n * 16, sbytes = (size_t)(k / 32) * n * 2;
    twm_weight *w = nullptr;
    if (pbytes == 0) {
        w = weight_from_device(ctx, nullptr, nullptr, k, n);
    } else {
        void *stage = nullptr;
        hipError_t e = hipMalloc(&stage, pbytes + sbytes);
        if (e != hipSuccess) { api_fail(TWM_MEMORY_ERROR, "twm_weight_gate_up: staging hipMalloc: %s", hipGetErrorString(e)); return nullptr; }
        uint8_t *p = (uint8_t *)stage;
        uint16_t *sc = (uint16_t *)(p + pbytes);
        if (twm_pair_gate_up(ctx, gate_packed_dev, gate_scales_dev, up_packed_dev, up_scales_dev, k, ffn_dim, p, sc) == TWM_OK)
            w = weight_from_device(ctx, p, sc, k, n);  // synchronises the stream before returning
        else
            (void)hipStreamSynchronize(ctx->stream);
        (void)hipFree(stage);
    }
    if (w) w->paired = true;
    return w;
}

int twm_weight_is_paired(const twm_weight *w) { return w && w->paired ? 1 : 0; }

void twm_weight_destroy(twm_weight *w)
{
    if (!w) return;
    if (w->qw || w->cq) (void)hipStreamSynchronize(w->ctx->stream);
    weight_release(w);
}

int twm_weight_dims(const twm_weight *w, uint32_t *k, uint32_t *n)
{
    if (!w) return api_fail(TWM_INVALID_HANDLE, "twm_weight_dims: null weight");
    if (k) *k = w->k;
    if (n) *n = w->n;
    return TWM_OK;
}

size_t twm_weight_bytes(const twm_weight *w) { return w ? w->bytes : 0; }

/* ---- repacked weights as a byte blob (for an on-disk cache) -------------------------------- */

// 64-byte little-endian header followed by the device allocation as it is.
struct WeightBlobHeader {
    char magic[8];          // "TWMWGT01"
    uint32_t layout;        // changes whenever the repacked byte order does
    uint32_t k, n, n_tiles, k_chunks;
    uint32_t paired;
    uint64_t payload_bytes;
    uint64_t checksum;      // of the payload
    uint8_t copies;         // payload: the 16-column tile copy (bit 0) and / or the column-lane copy (bit 1), in this order
    uint8_t reserved[15];
};
static_assert(sizeof(WeightBlobHeader) == 64, "blob header is 64 bytes");
static const char kBlobMagic[8] = {'T', 'W', 'M', 'W', 'G', 'T', '0', '1'};
static const uint32_t kBlobLayout = 5;
static const size_t kBlobTrailer = sizeof(TunedPlan) * kTuneBuckets;  // the measured plans (twm_weight_tune), after the payload

// Four independent multiply-rotate lanes over 64-bit words (memory-bound on the host), folded at the end.
static uint64_t blob_checksum(const uint8_t *p, size_t bytes)
{
    uint64_t h[4] = {0x9E3779B97F4A7C15ull, 0xC2B2AE3D27D4EB4Full, 0x165667B19E3779F9ull, 0x27D4EB2F165667C5ull};
    size_t words = bytes / 8, i = 0;
    for (; i + 4 <= words; i += 4) {
        for (int l = 0; l < 4; l++) {
            uint64_t v;
            memcpy(&v, p + (i + l) * 8, 8);
            h[l] = (h[l] ^ v) * 0x100000001B3ull;
            h[l] = (h[l] << 29) | (h[l] >> 35);
        }
    }
    uint64_t tail = 0;
    for (size_t b = i * 8; b < bytes; b++) tail = tail * 257 + p[b];
    uint64_t r = tail ^ (uint64_t)bytes;
    for (int l = 0; l < 4; l++) r = (r ^ h[l]) * 0xFF51AFD7ED558CCDull + (r >> 31);
    return r;
}

size_t twm_weight_blob_bytes(const twm_weight *w) { return w ? sizeof(WeightBlobHeader) + w->bytes + kBlobTrailer : 0; }

int twm_weight_export(twm_ctx *ctx, const twm_weight *w, void *blob_host, size_t blob_bytes)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "twm_weight_export: null handle");
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "twm_weight_export: weight belongs to another context");
    if (ctx->capturing) return api_fail(TWM_UNSUPPORTED_OP, "twm_weight_export: not allowed inside a graph capture");
    if (!blob_host) return api_fail(TWM_INVALID_HANDLE, "twm_weight_export: null buffer");
    if (blob_bytes != twm_weight_blob_bytes(w))
        return api_fail(TWM_SHAPE_ERROR, "twm_weight_export: the buffer must hold %zu bytes, got %zu", twm_weight_blob_bytes(w), blob_bytes);
    uint8_t *payload = (uint8_t *)blob_host + sizeof(WeightBlobHeader);
    size_t at = 0;
    if (w->qw) {
        if (int rc = twm_memcpy_d2h(ctx, payload + at, w->qw, w->copy_bytes)) return rc;
        at += w->copy_bytes;
    }
    if (w->cq) {
        if (int rc = twm_memcpy_d2h(ctx, payload + at, w->cq, w->copy_bytes)) return rc;
        at += w->copy_bytes;
    }
    WeightBlobHeader hd;
    memset(&hd, 0, sizeof hd);
    memcpy(hd.magic, kBlobMagic, 8);
    hd.layout = kBlobLayout;
    hd.k = w->k;
    hd.n = w->n;
    hd.n_tiles = w->n_tiles;
    hd.k_chunks = w->k_chunks;
    hd.paired = w->paired ? 1u : 0u;
    hd.payload_bytes = at;
    hd.checksum = blob_checksum(payload, at);
    hd.copies = (uint8_t)copies_of(w);
    memcpy(blob_host, &hd, sizeof hd);
    memcpy(payload + at, w->tuned, kBlobTrailer);
    return TWM_OK;
}

twm_weight *twm_weight_import(twm_ctx *ctx, const void *blob_host, size_t blob_bytes)
{
    if (!ctx) { api_fail(TWM_INVALID_HANDLE, "twm_weight_import: null context"); return nullptr; }
    if (ctx->capturing) { api_fail(TWM_UNSUPPORTED_OP, "twm_weight_import: not allowed inside a graph capture"); return nullptr; }
    if (!blob_host || blob_bytes < sizeof(WeightBlobHeader)) { api_fail(TWM_SHAPE_ERROR, "twm_weight_import: blob shorter than its header"); return nullptr; }
    WeightBlobHeader hd;
    memcpy(&hd, blob_host, sizeof hd);
    if (memcmp(hd.magic, kBlobMagic, 8) != 0) { api_fail(TWM_SHAPE_ERROR, "twm_weight_import: not a repacked-weight blob (bad magic)"); return nullptr; }
    if (hd.layout != kBlobLayout) {
        api_fail(TWM_UNSUPPORTED_OP, "twm_weight_import: blob has layout %u, this library writes %u: repack from the TW-Marlin arrays", hd.layout, kBlobLayout);
        return nullptr;
    }
    if (check_kn("twm_weight_import", hd.k, hd.n)) return nullptr;
    twm_weight *w = weight_alloc(ctx, hd.k, hd.n);
    if (!w) return nullptr;
    const uint8_t *payload = (const uint8_t *)blob_host + sizeof(WeightBlobHeader);
    const int held = hd.copies & 3, n_held = (held & 1) + (held >> 1);
    bool ok = w->n_tiles == hd.n_tiles && w->k_chunks == hd.k_chunks && hd.copies <= 3 &&
              (w->copy_bytes == 0 ? hd.payload_bytes == 0 : (n_held >= 1 && hd.payload_bytes == (uint64_t)n_held * w->copy_bytes)) &&
              blob_bytes == sizeof(WeightBlobHeader) + hd.payload_bytes + kBlobTrailer && hd.paired <= 1 &&
              (!hd.paired || hd.n % (2 * kPairWidth) == 0);
    if (!ok) api_fail(TWM_SHAPE_ERROR, "twm_weight_import: header does not describe a %u x %u weight of %zu bytes", hd.k, hd.n, blob_bytes);
    if (ok && blob_checksum(payload, (size_t)hd.payload_bytes) != hd.checksum) {
        ok = false;
        api_fail(TWM_SHAPE_ERROR, "twm_weight_import: checksum mismatch (corrupt or truncated blob)");
    }
    if (ok && w->copy_bytes) {
        ok = weight_alloc_copies(w, held, "twm_weight_import") == TWM_OK;
        size_t at = 0;
        if (ok && w->qw) { ok = twm_memcpy_h2d(ctx, w->qw, payload + at, w->copy_bytes) == TWM_OK; at += w->copy_bytes; }
        if (ok && w->cq) ok = twm_memcpy_h2d(ctx, w->cq, payload + at, w->copy_bytes) == TWM_OK;
    }
    if (!ok) {
        weight_release(w);
        return nullptr;
    }
    w->paired = hd.paired != 0;
    memcpy(w->tuned, payload + hd.payload_bytes, kBlobTrailer);
    for (TunedPlan &p : w->tuned)   // (a plan is a set of option values: anything outside their ranges is dropped)
        if (p.valid > 1 || p.kernel > 4 || p.kernel == 1 || p.nt > 4 || p.waves > 16 || p.sub_waves > 16 ||
            (p.sub != 0 && p.sub != 1 && p.sub != 16 && p.sub != 32) || (p.prefill_bm != 0 && p.prefill_bm != 64 && p.prefill_bm != 128 && p.prefill_bm != 192))
            memset(&p, 0, sizeof p);
    return w;
}

extern "C++" WeightView view_of(const twm_weight *w)
{
    WeightView v;
    v.qw = w->qw;
    v.sc = w->sc;
    v.cq = w->cq;
    v.k = w->k;
    v.n = w->n;
    v.groups = w->groups;
    v.n_tiles = w->n_tiles;
    v.k_chunks = w->k_chunks;
    return v;
}

int twm_weight_dequant_f16(twm_ctx *ctx, const twm_weight *w, uint16_t *out_kn_dev)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "twm_weight_dequant_f16: null handle");
    if ((uint64_t)w->k * w->n == 0) return TWM_OK;
    if (!out_kn_dev) return api_fail(TWM_INVALID_HANDLE, "twm_weight_dequant_f16: null output");
    // "dequant_src" = 1 reads the column-lane copy instead of the 16-column tile order (each builds its copy if need be)
    if (int rc = weight_ensure(ctx, w, ctx->dequant_src == 1 ? kCopyCol : kCopyTile, "twm_weight_dequant_f16")) return rc;
    if (ctx->dequant_src == 1)
        HIP_TRY(launch_weight_dequant_f16_col(ctx->stream, view_of(w), out_kn_dev), TWM_DEVICE_ERROR, "dequant launch");
    else
        HIP_TRY(launch_weight_dequant_f16(ctx->stream, view_of(w), out_kn_dev), TWM_DEVICE_ERROR, "dequant launch");
    return TWM_OK;
}

}  // extern "C"
