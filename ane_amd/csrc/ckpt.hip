// ckpt.hip — reader/writer for the training checkpoints of the two big loops, with device memory on the
// tensor side.
//
// File = CkptHdr (96 bytes; training/stories_config.h:90-105 for version 2, training/training_dynamic/config.h:78-86
// for version 4, where the three trailing pad ints carry kv_heads, head_dim, q_dim) followed by raw fp32 arrays
// in the order of save_checkpoint (training/train_large.m:110-146, training/training_dynamic/train.m:104-137):
//   per layer: Wq Wk Wv Wo W1 W2 W3 rms_att rms_ffn, then (m, v) of each of those nine in the same order;
//   then rms_final, its m, v; then embed, its m, v.
// Sizes: Wq = q_dim*dim, Wk = Wv = kv_dim*dim, Wo = dim*q_dim, W1 = W3 = hidden*dim, W2 = dim*hidden, norms = dim,
// embed = vocab*dim; version 2 is the multi-head case q_dim = kv_dim = dim.
// The header and the index are host-only code and work without a GPU; load/store stream through one pinned
// staging buffer.
#include "common.h"

#include <errno.h>

namespace {

constexpr int CK_MAGIC = 0x424C5A54;
constexpr size_t STAGE_BYTES = 32u << 20;
void *g_stage = nullptr;

struct Dims {
    uint64_t dim, hidden, q_dim, kv_dim, vocab, layers;
};

int dims_of(const mi355_ckpt_hdr *h, Dims *d) {
    if (!h) return mi355_fail("ckpt: NULL header");
    if (h->magic != CK_MAGIC) return mi355_fail("ckpt: bad magic 0x%08x", (unsigned)h->magic);
    if (h->version != 2 && h->version != 4) return mi355_fail("ckpt: unsupported version %d", h->version);
    if (h->n_layers <= 0 || h->vocab_size <= 0 || h->dim <= 0 || h->hidden_dim <= 0 || h->n_heads <= 0)
        return mi355_fail("ckpt: bad model shape in header");
    d->dim = (uint64_t)h->dim;
    d->hidden = (uint64_t)h->hidden_dim;
    d->vocab = (uint64_t)h->vocab_size;
    d->layers = (uint64_t)h->n_layers;
    if (h->version == 4) {
        if (h->kv_heads <= 0 || h->head_dim <= 0 || h->q_dim <= 0) return mi355_fail("ckpt: bad GQA fields in header");
        d->q_dim = (uint64_t)h->q_dim;
        d->kv_dim = (uint64_t)h->kv_heads * (uint64_t)h->head_dim;
    } else {
        d->q_dim = d->kv_dim = d->dim;
    }
    return 0;
}

// element counts of the nine per-layer tensors, in file order
void layer_counts(const Dims &d, uint64_t (&n)[9]) {
    n[MI355_CK_WQ] = d.q_dim * d.dim;
    n[MI355_CK_WK] = d.kv_dim * d.dim;
    n[MI355_CK_WV] = d.kv_dim * d.dim;
    n[MI355_CK_WO] = d.dim * d.q_dim;
    n[MI355_CK_W1] = d.hidden * d.dim;
    n[MI355_CK_W2] = d.dim * d.hidden;
    n[MI355_CK_W3] = d.hidden * d.dim;
    n[MI355_CK_RMS_ATT] = d.dim;
    n[MI355_CK_RMS_FFN] = d.dim;
}

void *stage() {
    if (!g_stage && hipHostMalloc(&g_stage, STAGE_BYTES, hipHostMallocDefault) != hipSuccess) {
        g_stage = nullptr;
        mi355_fail("ckpt: cannot allocate the pinned staging buffer");
    }
    return g_stage;
}

}   // namespace

void mi355_ckpt_free(void) {
    if (g_stage) (void)hipHostFree(g_stage);
    g_stage = nullptr;
}

static_assert(sizeof(mi355_ckpt_hdr) == 96, "checkpoint header is 96 bytes on disk");

MI355_API int mi355_ckpt_read_header(const char *path, mi355_ckpt_hdr *hdr) {
    if (!path || !hdr) return mi355_fail("ckpt_read_header: NULL argument");
    FILE *f = fopen(path, "rb");
    if (!f) return mi355_fail("ckpt_read_header: %s: %s", path, strerror(errno));
    mi355_ckpt_hdr h;
    const size_t got = fread(&h, 1, sizeof(h), f);
    fclose(f);
    if (got != sizeof(h)) return mi355_fail("ckpt_read_header: %s: shorter than a header", path);
    Dims d;
    if (dims_of(&h, &d)) return -1;
    *hdr = h;
    return 0;
}

MI355_API int mi355_ckpt_locate(const mi355_ckpt_hdr *hdr, int layer, int tensor, int part, uint64_t *byte_offset,
                                uint64_t *count) {
    Dims d;
    if (dims_of(hdr, &d)) return -1;
    if (part < MI355_CK_WEIGHT || part > MI355_CK_ADAM_V) return mi355_fail("ckpt_locate: part must be 0, 1 or 2");
    uint64_t n[9];
    layer_counts(d, n);
    uint64_t per_layer = 0;
    for (uint64_t c : n) per_layer += 3 * c;
    uint64_t off = sizeof(mi355_ckpt_hdr) / 4, cnt;    // in floats
    if (tensor >= MI355_CK_WQ && tensor <= MI355_CK_RMS_FFN) {
        if (layer < 0 || (uint64_t)layer >= d.layers) return mi355_fail("ckpt_locate: layer %d outside 0..%d", layer, (int)d.layers - 1);
        off += (uint64_t)layer * per_layer;
        if (part == MI355_CK_WEIGHT) {
            for (int t = 0; t < tensor; t++) off += n[t];
        } else {
            for (uint64_t c : n) off += c;                      // past the nine weights
            for (int t = 0; t < tensor; t++) off += 2 * n[t];   // (m, v) pairs before this tensor
            if (part == MI355_CK_ADAM_V) off += n[tensor];
        }
        cnt = n[tensor];
    } else if (tensor == MI355_CK_RMS_FINAL || tensor == MI355_CK_EMBED) {
        off += d.layers * per_layer;
        cnt = d.dim;
        if (tensor == MI355_CK_EMBED) {
            off += 3 * d.dim;
            cnt = d.vocab * d.dim;
        }
        off += (uint64_t)part * cnt;
    } else {
        return mi355_fail("ckpt_locate: unknown tensor %d", tensor);
    }
    if (byte_offset) *byte_offset = off * 4;
    if (count) *count = cnt;
    return 0;
}

MI355_API uint64_t mi355_ckpt_file_bytes(const mi355_ckpt_hdr *hdr) {
    uint64_t off = 0, cnt = 0;
    if (mi355_ckpt_locate(hdr, 0, MI355_CK_EMBED, MI355_CK_ADAM_V, &off, &cnt)) return 0;
    return off + cnt * 4;
}

MI355_API int mi355_ckpt_create(const char *path, const mi355_ckpt_hdr *hdr) {
    if (!path) return mi355_fail("ckpt_create: NULL path");
    const uint64_t total = mi355_ckpt_file_bytes(hdr);
    if (!total) return -1;
    FILE *f = fopen(path, "wb");
    if (!f) return mi355_fail("ckpt_create: %s: %s", path, strerror(errno));
    bool ok = fwrite(hdr, 1, sizeof(*hdr), f) == sizeof(*hdr);
    // size the file now, so that tensors can be stored in any order
    ok = ok && fseeko(f, (off_t)total - 1, SEEK_SET) == 0 && fputc(0, f) != EOF;
    ok = (fclose(f) == 0) && ok;
    if (!ok) return mi355_fail("ckpt_create: %s: write failed", path);
    return 0;
}

MI355_API int mi355_ckpt_load_dev(const char *path, uint64_t byte_offset, float *dst_dev, uint64_t count) {
    if (!mi355_ready("ckpt_load") || !mi355_outside_capture("ckpt_load")) return -1;
    if (!path || !dst_dev) return mi355_fail("ckpt_load: NULL argument");
    char *buf = (char *)stage();
    if (!buf) return -1;
    FILE *f = fopen(path, "rb");
    if (!f) return mi355_fail("ckpt_load: %s: %s", path, strerror(errno));
    if (fseeko(f, (off_t)byte_offset, SEEK_SET)) {
        fclose(f);
        return mi355_fail("ckpt_load: %s: cannot seek to %llu", path, (unsigned long long)byte_offset);
    }
    uint64_t left = count * 4, done = 0;
    while (left) {
        const size_t n = left < STAGE_BYTES ? (size_t)left : STAGE_BYTES;
        if (fread(buf, 1, n, f) != n) {
            fclose(f);
            return mi355_fail("ckpt_load: %s: file ends inside the tensor", path);
        }
        // the staging buffer is reused by the next piece: the copy must have finished before it is overwritten
        hipError_t e = hipMemcpyAsync((char *)dst_dev + done, buf, n, hipMemcpyHostToDevice, g_ctx.stream);
        if (e == hipSuccess) e = hipStreamSynchronize(g_ctx.stream);
        if (e != hipSuccess) {
            fclose(f);
            return mi355_fail("ckpt_load: copy to the device: %s", hipGetErrorString(e));
        }
        left -= n;
        done += n;
    }
    fclose(f);
    return 0;
}

MI355_API int mi355_ckpt_store_dev(const char *path, uint64_t byte_offset, const float *src_dev, uint64_t count) {
    if (!mi355_ready("ckpt_store") || !mi355_outside_capture("ckpt_store")) return -1;
    if (!path || !src_dev) return mi355_fail("ckpt_store: NULL argument");
    char *buf = (char *)stage();
    if (!buf) return -1;
    FILE *f = fopen(path, "r+b");
    if (!f) return mi355_fail("ckpt_store: %s: %s (create it with mi355_ckpt_create first)", path, strerror(errno));
    if (fseeko(f, (off_t)byte_offset, SEEK_SET)) {
        fclose(f);
        return mi355_fail("ckpt_store: %s: cannot seek to %llu", path, (unsigned long long)byte_offset);
    }
    uint64_t left = count * 4, done = 0;
    while (left) {
        const size_t n = left < STAGE_BYTES ? (size_t)left : STAGE_BYTES;
        hipError_t e = hipMemcpyAsync(buf, (const char *)src_dev + done, n, hipMemcpyDeviceToHost, g_ctx.stream);
        if (e == hipSuccess) e = hipStreamSynchronize(g_ctx.stream);
        if (e != hipSuccess) {
            fclose(f);
            return mi355_fail("ckpt_store: copy from the device: %s", hipGetErrorString(e));
        }
        if (fwrite(buf, 1, n, f) != n) {
            fclose(f);
            return mi355_fail("ckpt_store: %s: write failed", path);
        }
        left -= n;
        done += n;
    }
    if (fclose(f)) return mi355_fail("ckpt_store: %s: close failed", path);
    return 0;
}
