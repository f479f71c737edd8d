// Host side of the library: ternarise+pack producer, .tllm reader (into one device pool) and a
// synthetic-model writer. No kernels here; the only GPU calls are the copies of the upload.
#include <math.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <new>
#include <string>
#include <vector>

#include "../../include/tllm_model_file.h"
#include "common.h"

namespace {

constexpr uint32_t kMagic = 0x544C4C4Du;  // "TLLM" (reference include/format.h:8)
constexpr uint32_t kVersion = 1;
constexpr uint64_t kPoolAlign = 256;

uint16_t half_bits(float v) {  // round to nearest even
    const _Float16 h = (_Float16)v;
    uint16_t b;
    memcpy(&b, &h, 2);
    return b;
}

int pad32(int v) { return (v + 31) / 32 * 32; }  // reference src/model.cpp:63-65

struct Rng {  // splitmix64 + Box-Muller; only the synthetic writer uses it
    uint64_t s;
    uint64_t next() {
        uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double uniform() { return ((double)(next() >> 11) + 0.5) * (1.0 / 9007199254740992.0); }
    float normal() {
        const double u = uniform(), v = uniform();
        return (float)(sqrt(-2.0 * log(u)) * cos(6.283185307179586 * v));
    }
};

}  // namespace

struct tllm_model_file {
    std::string path;
    tllm_file_header header;
    std::vector<tllm_file_linear> linears;
    uint64_t pool_bytes = 0;
    uint64_t file_bytes = 0;  // through the last weight array (the tokenizer blob follows)
};

extern "C" {

int tllm_ternarize_pack_f32(const float *weight, int rows, int cols, int group_size, float threshold_factor,
                            uint32_t *nonzero_masks, uint32_t *sign_masks, uint16_t *scales) {
    if (!weight || !nonzero_masks || !sign_masks || !scales) return TLLM_ERR_NULL_POINTER;
    if (rows < 1 || cols < 1 || cols % 32 != 0) return TLLM_ERR_BAD_SHAPE;
    if (group_size < 32 || group_size % 32 != 0 || cols % group_size != 0) return TLLM_ERR_BAD_GROUP;
    const int words = cols / 32, groups = cols / group_size;
    for (int r = 0; r < rows; r++) {
        const float *row = weight + (size_t)r * cols;
        uint32_t *nz_row = nonzero_masks + (size_t)r * words;
        uint32_t *sg_row = sign_masks + (size_t)r * words;
        for (int g = 0; g < groups; g++) {
            const float *p = row + (size_t)g * group_size;
            float sum_abs = 0.0f;
            for (int j = 0; j < group_size; j++) sum_abs += fabsf(p[j]);
            const float thr = threshold_factor * (sum_abs / (float)group_size);
            float nz_sum = 0.0f;
            int nz_cnt = 0;
            for (int w = 0; w < group_size / 32; w++) {
                uint32_t nz = 0, sg = 0;
                for (int b = 0; b < 32; b++) {  // bit b of a word <-> column 32*word + b (LSB first)
                    const float v = p[32 * w + b];
                    if (v > thr) {
                        nz |= 1u << b;
                        sg |= 1u << b;
                        nz_sum += fabsf(v);
                        nz_cnt++;
                    } else if (v < -thr) {
                        nz |= 1u << b;
                        nz_sum += fabsf(v);
                        nz_cnt++;
                    }
                }
                nz_row[g * (group_size / 32) + w] = nz;
                sg_row[g * (group_size / 32) + w] = sg;
            }
            scales[(size_t)r * groups + g] = half_bits(nz_sum / (float)(nz_cnt > 0 ? nz_cnt : 1));
        }
    }
    return TLLM_OK;
}

int tllm_model_file_open(const char *path, tllm_model_file **file) {
    if (!path || !file) return TLLM_ERR_NULL_POINTER;
    *file = nullptr;
    FILE *f = fopen(path, "rb");
    if (!f) return TLLM_ERR_IO;
    tllm_file_header h;
    const bool ok = fread(&h, sizeof h, 1, f) == 1;
    uint64_t size = 0;
    if (ok && fseek(f, 0, SEEK_END) == 0) size = (uint64_t)ftell(f);
    fclose(f);
    if (!ok) return TLLM_ERR_IO;
    if (h.magic != kMagic || h.version != kVersion) return TLLM_ERR_BAD_FILE;
    // Every size is bounded BEFORE any arithmetic on it: the fields come from an untrusted file, and an
    // overflowed product would pass the truncation check below and send uploads to wild pool offsets.
    constexpr uint32_t kMaxDim = 1u << 24;       // rows or columns of one matrix
    constexpr uint64_t kMaxElems = 1ull << 40;   // weights of one matrix, vocabulary table elements
    if (!h.vocab_size || !h.hidden_dim || !h.intermediate_dim || !h.n_heads || !h.n_kv_heads || !h.head_dim ||
        h.group_size < 32 || h.group_size % 32 != 0 || h.group_size > kMaxDim || h.n_layers > 4096 ||
        h.vocab_size > kMaxDim || h.hidden_dim > kMaxDim || h.intermediate_dim > kMaxDim || h.n_heads > kMaxDim ||
        h.n_kv_heads > kMaxDim || h.head_dim > kMaxDim)
        return TLLM_ERR_BAD_FILE;
    const uint64_t q64 = (uint64_t)h.n_heads * h.head_dim, kv64 = (uint64_t)h.n_kv_heads * h.head_dim;
    if (q64 > kMaxDim || kv64 > kMaxDim) return TLLM_ERR_BAD_FILE;
    const int gs = (int)h.group_size;
    const int hidden_pad = pad32((int)h.hidden_dim);
    const int q_dim = (int)q64, kv_dim = (int)kv64;
    const int q_pad = pad32(q_dim), inter_pad = pad32((int)h.intermediate_dim);
    if (hidden_pad % gs || q_pad % gs || inter_pad % gs) return TLLM_ERR_BAD_FILE;
    {
        const uint64_t widest = (uint64_t)std::max(std::max(hidden_pad, q_pad), inter_pad);
        const uint64_t tallest = std::max<uint64_t>(std::max<uint64_t>(h.intermediate_dim, h.vocab_size), std::max<uint64_t>(q64, h.hidden_dim));
        if (widest * tallest > kMaxElems) return TLLM_ERR_BAD_FILE;   // with <= 4096 layers x 7 matrices the sums stay below 2^63
    }

    tllm_model_file *m = new (std::nothrow) tllm_model_file;
    if (!m) return TLLM_ERR_TOO_LARGE;
    m->path = path;
    m->header = h;
    uint64_t pos = sizeof h, pool = 0;
    pos += (uint64_t)h.vocab_size * h.hidden_dim * 2;  // fp16 embedding table
    auto add = [&](int rows, int cols, int layer, int kind) {
        tllm_file_linear l{};
        const uint64_t mask_bytes = (uint64_t)rows * (cols / 32) * 4, scale_bytes = (uint64_t)rows * (cols / gs) * 2;
        auto up = [](uint64_t v) { return (v + kPoolAlign - 1) / kPoolAlign * kPoolAlign; };
        l.nonzero_file = pos;
        l.sign_file = pos + mask_bytes;
        l.scales_file = pos + 2 * mask_bytes;
        pos += 2 * mask_bytes + scale_bytes;
        l.nonzero_pool = pool;
        l.sign_pool = pool + up(mask_bytes);
        l.scales_pool = pool + 2 * up(mask_bytes);
        pool += 2 * up(mask_bytes) + up(scale_bytes);
        l.rows = rows;
        l.cols = cols;
        l.layer = layer;
        l.kind = kind;
        m->linears.push_back(l);
    };
    for (uint32_t i = 0; i < h.n_layers; i++) {
        add(q_dim, hidden_pad, (int)i, 0);
        add(kv_dim, hidden_pad, (int)i, 1);
        add(kv_dim, hidden_pad, (int)i, 2);
        add((int)h.hidden_dim, q_pad, (int)i, 3);
        add((int)h.intermediate_dim, hidden_pad, (int)i, 4);
        add((int)h.intermediate_dim, hidden_pad, (int)i, 5);
        add((int)h.hidden_dim, inter_pad, (int)i, 6);
        pos += 2 * (uint64_t)h.hidden_dim * 2;  // attention and FFN norm weights (fp16)
    }
    pos += (uint64_t)h.hidden_dim * 2;  // final norm
    if (h.flags & 1u) add((int)h.vocab_size, hidden_pad, -1, 7);
    else pos += (uint64_t)h.vocab_size * h.hidden_dim * 2;
    m->pool_bytes = pool;
    m->file_bytes = pos;
    if (size < pos) {
        delete m;
        return TLLM_ERR_IO;  // truncated
    }
    *file = m;
    return TLLM_OK;
}

void tllm_model_file_close(tllm_model_file *file) { delete file; }

int tllm_model_file_header(const tllm_model_file *file, tllm_file_header *header) {
    if (!file || !header) return TLLM_ERR_NULL_POINTER;
    *header = file->header;
    return TLLM_OK;
}

int tllm_model_file_linear_count(const tllm_model_file *file) { return file ? (int)file->linears.size() : TLLM_ERR_NULL_POINTER; }

int tllm_model_file_linear(const tllm_model_file *file, int index, tllm_file_linear *out) {
    if (!file || !out) return TLLM_ERR_NULL_POINTER;
    if (index < 0 || index >= (int)file->linears.size()) return TLLM_ERR_BAD_SHAPE;
    *out = file->linears[index];
    return TLLM_OK;
}

uint64_t tllm_model_file_pool_bytes(const tllm_model_file *file) { return file ? file->pool_bytes : 0; }

int tllm_model_file_upload(const tllm_model_file *file, void *device_pool, uint64_t pool_bytes, tllm_stream_t stream) {
    if (!file || !device_pool) return TLLM_ERR_NULL_POINTER;
    if (pool_bytes < file->pool_bytes) return TLLM_ERR_TOO_LARGE;
    if (reinterpret_cast<uintptr_t>(device_pool) % kPoolAlign) return TLLM_ERR_MISALIGNED;
    FILE *f = fopen(file->path.c_str(), "rb");
    if (!f) return TLLM_ERR_IO;
    constexpr size_t kStage = (size_t)32 << 20;  // two pinned halves of 16 MiB, used alternately
    char *stage = nullptr;
    if (hipError_t e = hipHostMalloc(reinterpret_cast<void **>(&stage), kStage, hipHostMallocDefault)) {
        fclose(f);
        return (int)e;
    }
    hipStream_t s = (hipStream_t)stream;
    int rc = TLLM_OK;
    int half = 0;
    hipEvent_t done[2] = {nullptr, nullptr};
    bool used[2] = {false, false};
    for (int i = 0; i < 2 && rc == TLLM_OK; i++)
        if (hipError_t e = hipEventCreateWithFlags(&done[i], hipEventDisableTiming)) rc = (int)e;
    auto copy_array = [&](uint64_t file_off, uint64_t pool_off, uint64_t bytes) {
        if (fseek(f, (long)file_off, SEEK_SET) != 0) {
            rc = TLLM_ERR_IO;
            return;
        }
        while (bytes && rc == TLLM_OK) {
            const size_t n = bytes < kStage / 2 ? (size_t)bytes : kStage / 2;
            char *buf = stage + (size_t)half * (kStage / 2);
            if (used[half])
                if (hipError_t e = hipEventSynchronize(done[half])) rc = (int)e;  // the copy that last used this half
            if (rc == TLLM_OK && fread(buf, 1, n, f) != n) rc = TLLM_ERR_IO;
            if (rc == TLLM_OK)
                if (hipError_t e = hipMemcpyAsync(static_cast<char *>(device_pool) + pool_off, buf, n, hipMemcpyHostToDevice, s))
                    rc = (int)e;
            if (rc == TLLM_OK)
                if (hipError_t e = hipEventRecord(done[half], s)) rc = (int)e;
            used[half] = true;
            half ^= 1;
            pool_off += n;
            bytes -= n;
        }
    };
    const uint64_t gs = file->header.group_size;
    for (const tllm_file_linear &l : file->linears) {
        if (rc != TLLM_OK) break;
        const uint64_t mask_bytes = (uint64_t)l.rows * (l.cols / 32) * 4, scale_bytes = (uint64_t)l.rows * (l.cols / gs) * 2;
        copy_array(l.nonzero_file, l.nonzero_pool, mask_bytes);
        copy_array(l.sign_file, l.sign_pool, mask_bytes);
        copy_array(l.scales_file, l.scales_pool, scale_bytes);
    }
    if (hipError_t e = hipStreamSynchronize(s))
        if (rc == TLLM_OK) rc = (int)e;
    for (int i = 0; i < 2; i++)
        if (done[i]) (void)hipEventDestroy(done[i]);
    (void)hipHostFree(stage);
    fclose(f);
    return rc;
}

int tllm_model_file_problem(const tllm_model_file *file, int index, void *device_pool, tllm_linear_problem *problem) {
    if (!file || !device_pool || !problem) return TLLM_ERR_NULL_POINTER;
    if (index < 0 || index >= (int)file->linears.size()) return TLLM_ERR_BAD_SHAPE;
    const tllm_file_linear &l = file->linears[index];
    char *base = static_cast<char *>(device_pool);
    problem->nonzero_masks = reinterpret_cast<const uint32_t *>(base + l.nonzero_pool);
    problem->sign_masks = reinterpret_cast<const uint32_t *>(base + l.sign_pool);
    problem->scales = reinterpret_cast<const uint16_t *>(base + l.scales_pool);
    problem->rows = l.rows;
    problem->cols = l.cols;
    return TLLM_OK;
}

int tllm_model_file_write_synthetic(const char *path, const tllm_file_header *header, uint64_t seed) {
    if (!path || !header) return TLLM_ERR_NULL_POINTER;
    tllm_file_header h = *header;
    h.magic = kMagic;
    h.version = kVersion;
    memset(h.reserved, 0, sizeof h.reserved);
    const int gs = (int)h.group_size;
    if (!h.vocab_size || !h.hidden_dim || !h.intermediate_dim || !h.n_heads || !h.n_kv_heads || !h.head_dim ||
        gs < 32 || gs % 32 != 0)
        return TLLM_ERR_BAD_FILE;
    const int hidden = (int)h.hidden_dim, q_dim = (int)(h.n_heads * h.head_dim), kv_dim = (int)(h.n_kv_heads * h.head_dim);
    const int inter = (int)h.intermediate_dim;
    if (hidden % gs || q_dim % gs || inter % gs) return TLLM_ERR_BAD_GROUP;
    FILE *f = fopen(path, "wb");
    if (!f) return TLLM_ERR_IO;
    Rng rng{seed * 0x9E3779B97F4A7C15ull + 1};
    bool ok = fwrite(&h, sizeof h, 1, f) == 1;
    auto write_fp16 = [&](size_t count, float scale, float offset) {
        std::vector<uint16_t> buf(count);
        for (size_t i = 0; i < count; i++) buf[i] = half_bits(offset + scale * rng.normal());
        ok = ok && fwrite(buf.data(), 2, count, f) == count;
    };
    auto write_linear = [&](int rows, int cols) {
        std::vector<float> w((size_t)rows * cols);
        for (float &v : w) v = 0.02f * rng.normal();
        std::vector<uint32_t> nz((size_t)rows * (cols / 32)), sg(nz.size());
        std::vector<uint16_t> sc((size_t)rows * (cols / gs));
        ok = ok && tllm_ternarize_pack_f32(w.data(), rows, cols, gs, 0.7f, nz.data(), sg.data(), sc.data()) == TLLM_OK;
        ok = ok && fwrite(nz.data(), 4, nz.size(), f) == nz.size();
        ok = ok && fwrite(sg.data(), 4, sg.size(), f) == sg.size();
        ok = ok && fwrite(sc.data(), 2, sc.size(), f) == sc.size();
    };
    write_fp16((size_t)h.vocab_size * hidden, 0.02f, 0.0f);  // embedding table
    for (uint32_t i = 0; i < h.n_layers && ok; i++) {
        write_linear(q_dim, hidden);
        write_linear(kv_dim, hidden);
        write_linear(kv_dim, hidden);
        write_linear(hidden, q_dim);
        write_linear(inter, hidden);
        write_linear(inter, hidden);
        write_linear(hidden, inter);
        write_fp16((size_t)hidden, 0.05f, 1.0f);  // attention norm
        write_fp16((size_t)hidden, 0.05f, 1.0f);  // FFN norm
    }
    write_fp16((size_t)hidden, 0.05f, 1.0f);  // final norm
    if (h.flags & 1u) write_linear((int)h.vocab_size, hidden);
    else write_fp16((size_t)h.vocab_size * hidden, 0.02f, 0.0f);
    const uint64_t tok_size = 0;  // no tokenizer blob
    ok = ok && fwrite(&tok_size, 8, 1, f) == 1;
    ok = (fclose(f) == 0) && ok;
    return ok ? TLLM_OK : TLLM_ERR_IO;
}

}  // extern "C"
