// Checkpoint files to weights: safetensors (one file or a directory of shards) and GGUF v2 / v3, read through
// mmap; the tensor-name maps of the reference's Qwen3 / Gemma3 loaders; upload of a tensor as a WMat with the
// conversion done on the GPU.  Interface and reference citations: include/loader_hip.h.
#include "backend.h"
#include "devutil.h"
#include "../../include/loader_hip.h"

#include <algorithm>
#include <dirent.h>
#include <fcntl.h>
#include <map>
#include <math.h>
#include <string.h>
#include <string>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>
#include <vector>

using namespace lmhip;

namespace {

struct Mapping {
    void *p = nullptr;
    size_t size = 0;
    size_t data_off = 0;          // first byte of tensor data
};

struct TensorInfo {
    std::string name;
    int dtype = -1, ndim = 0, shard = 0;
    uint64_t shape[4] = {0, 0, 0, 0};
    uint64_t begin = 0, nbytes = 0;   // relative to the shard's data_off
    // Product of the dimensions; UINT64_MAX when it would pass 2^48 (no tensor of a model file is that large, and
    // nothing downstream can then overflow when it multiplies by an element size).
    uint64_t elements() const
    {
        constexpr uint64_t cap = (uint64_t)1 << 48;
        uint64_t n = 1;
        for (int d = 0; d < ndim; d++) {
            if (shape[d] != 0 && n > cap / shape[d]) return UINT64_MAX;
            n *= shape[d];
        }
        return n;
    }
};

// true when [begin, begin + nbytes) lies inside the data section of a mapping of `size` bytes that starts at data_off
// (written so that no sum can wrap)
bool range_inside(uint64_t data_off, uint64_t begin, uint64_t nbytes, uint64_t size)
{
    return data_off <= size && begin <= size - data_off && nbytes <= size - data_off - begin;
}

}  // namespace

struct ModelFile {
    bool gguf = false;
    std::vector<Mapping> maps;
    std::vector<TensorInfo> tensors;
    std::map<std::string, int> index;
};

namespace {

bool map_file(const std::string &path, Mapping &m)
{
    const int fd = open(path.c_str(), O_RDONLY);
    if (fd < 0) return false;
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size < 8) { close(fd); return false; }
    m.size = (size_t)st.st_size;
    m.p = mmap(nullptr, m.size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (m.p == MAP_FAILED) { m.p = nullptr; return false; }
    return true;
}

size_t bytes_of(int dtype, uint64_t n)
{
    switch (dtype) {
    case MF_F32: return n * 4;
    case MF_F16: case MF_BF16: return n * 2;
    case MF_Q8_0: return (n + 31) / 32 * 34;
    default: return 0;
    }
}

// ---------------------------------------------------------------- safetensors header (JSON)

// A cursor over the header text.  The header is one object: tensor name -> {"dtype", "shape", "data_offsets"}, plus
// an optional "__metadata__" object of strings.
struct Json {
    const char *p, *end;
    void ws() { while (p < end && (*p == ' ' || *p == '\n' || *p == '\r' || *p == '\t')) p++; }
    bool eat(char c) { ws(); if (p < end && *p == c) { p++; return true; } return false; }
    bool string(std::string &out)
    {
        ws();
        if (p >= end || *p != '"') return false;
        out.clear();
        for (p++; p < end && *p != '"'; p++) {
            if (*p == '\\' && p + 1 < end) p++;
            out.push_back(*p);
        }
        if (p >= end) return false;
        p++;
        return true;
    }
    bool number(uint64_t &v)
    {
        ws();
        if (p >= end || *p < '0' || *p > '9') return false;
        v = 0;
        while (p < end && *p >= '0' && *p <= '9') v = v * 10 + (uint64_t)(*p++ - '0');
        return true;
    }
    bool skip()                    // any value
    {
        ws();
        if (p >= end) return false;
        if (*p == '"') { std::string s; return string(s); }
        if (*p == '{' || *p == '[') {
            const char open = *p, close = open == '{' ? '}' : ']';
            p++;
            if (eat(close)) return true;
            do {
                if (open == '{') { std::string k; if (!string(k) || !eat(':')) return false; }
                if (!skip()) return false;
            } while (eat(','));
            return eat(close);
        }
        while (p < end && *p != ',' && *p != '}' && *p != ']') p++;
        return true;
    }
};

bool parse_safetensors_header(const char *text, size_t len, int shard, std::vector<TensorInfo> &out)
{
    Json j{text, text + len};
    if (!j.eat('{')) return false;
    if (j.eat('}')) return true;
    do {
        std::string name;
        if (!j.string(name) || !j.eat(':')) return false;
        if (name == "__metadata__") { if (!j.skip()) return false; continue; }
        if (!j.eat('{')) return false;
        TensorInfo t;
        t.name = name; t.shard = shard;
        uint64_t off[2] = {0, 0};
        if (!j.eat('}')) {
            do {
                std::string field;
                if (!j.string(field) || !j.eat(':')) return false;
                if (field == "dtype") {
                    std::string d;
                    if (!j.string(d)) return false;
                    t.dtype = d == "F32" ? MF_F32 : d == "F16" ? MF_F16 : d == "BF16" ? MF_BF16 : -1;
                } else if (field == "shape" || field == "data_offsets") {
                    if (!j.eat('[')) return false;
                    int n = 0;
                    uint64_t v;
                    while (j.number(v)) {
                        if (field == "shape") { if (n < 4) t.shape[n] = v; } else if (n < 2) off[n] = v;
                        n++;
                        if (!j.eat(',')) break;
                    }
                    if (!j.eat(']')) return false;
                    if (field == "shape") { if (n > 4) return false; t.ndim = n; }
                } else if (!j.skip()) return false;
            } while (j.eat(','));
            if (!j.eat('}')) return false;
        }
        if (off[1] < off[0]) return false;                 // reversed data_offsets
        t.begin = off[0];
        t.nbytes = off[1] - off[0];
        out.push_back(t);
    } while (j.eat(','));
    return j.eat('}');
}

bool open_safetensors_shard(const std::string &path, ModelFile *f)
{
    Mapping m;
    if (!map_file(path, m)) { fprintf(stderr, "[Loader] cannot map %s\n", path.c_str()); return false; }
    uint64_t hdr = 0;
    memcpy(&hdr, m.p, 8);
    if (hdr > m.size - 8) { fprintf(stderr, "[Loader] %s: header length %llu beyond the file\n", path.c_str(), (unsigned long long)hdr); munmap(m.p, m.size); return false; }
    m.data_off = 8 + hdr;
    const int shard = (int)f->maps.size();
    const size_t before = f->tensors.size();
    if (!parse_safetensors_header((const char *)m.p + 8, hdr, shard, f->tensors)) {
        fprintf(stderr, "[Loader] %s: malformed safetensors header\n", path.c_str());
        f->tensors.resize(before);
        munmap(m.p, m.size);
        return false;
    }
    for (size_t i = before; i < f->tensors.size(); i++) {
        const TensorInfo &t = f->tensors[i];
        const uint64_t ne = t.elements();
        if (ne == UINT64_MAX || !range_inside(m.data_off, t.begin, t.nbytes, m.size) || (t.dtype >= 0 && t.nbytes != bytes_of(t.dtype, ne))) {
            fprintf(stderr, "[Loader] %s: tensor %s has offsets outside the file or not matching its shape\n", path.c_str(), t.name.c_str());
            f->tensors.resize(before);
            munmap(m.p, m.size);
            return false;
        }
    }
    f->maps.push_back(m);
    return true;
}

// ---------------------------------------------------------------- GGUF

struct Reader {
    const uint8_t *p;
    size_t off, size;
    bool ok = true;
    template <typename T> T get() { T v{}; if (off + sizeof(T) > size) { ok = false; return v; } memcpy(&v, p + off, sizeof(T)); off += sizeof(T); return v; }
    std::string str() { const uint64_t n = get<uint64_t>(); if (!ok || n > size - off) { ok = false; return ""; } std::string s((const char *)p + off, n); off += n; return s; }
    void skip(uint64_t n) { if (n > size - off) ok = false; else off += n; }   // off <= size always, so the difference cannot wrap
};

// GGUF metadata value types (src/data/gguf.h:13-25): sizes of the scalar ones, 8 = string, 9 = array
void skip_gguf_value(Reader &r, uint32_t type, uint32_t *u32_out = nullptr)
{
    static const int scalar[13] = {1, 1, 2, 2, 4, 4, 4, 1, 0, 0, 8, 8, 8};
    if (type == 8) { r.str(); return; }
    if (type == 9) {
        const uint32_t et = r.get<uint32_t>();
        const uint64_t n = r.get<uint64_t>();
        if (et < 13 && scalar[et]) { if (n > r.size) r.ok = false; else r.skip(n * (uint64_t)scalar[et]); return; }
        for (uint64_t i = 0; i < n && r.ok; i++) skip_gguf_value(r, et);
        return;
    }
    if (type >= 13) { fprintf(stderr, "[Loader] GGUF: unknown metadata type %u\n", type); r.ok = false; return; }
    if (type == 4 && u32_out) { *u32_out = r.get<uint32_t>(); return; }
    r.skip(scalar[type]);
}

bool open_gguf(const std::string &path, ModelFile *f)
{
    Mapping m;
    if (!map_file(path, m)) { fprintf(stderr, "[Loader] cannot map %s\n", path.c_str()); return false; }
    Reader r{(const uint8_t *)m.p, 0, m.size};
    const uint32_t magic = r.get<uint32_t>(), version = r.get<uint32_t>();
    if (magic != 0x46554747u || version < 2 || version > 3) {
        fprintf(stderr, "[Loader] %s: not a GGUF v2 / v3 file (magic 0x%08X, version %u)\n", path.c_str(), magic, version);
        munmap(m.p, m.size);
        return false;
    }
    const uint64_t n_tensors = r.get<uint64_t>(), n_kv = r.get<uint64_t>();
    uint32_t alignment = 32;                                   // src/data/gguf.c:170; files may override it
    for (uint64_t i = 0; i < n_kv && r.ok; i++) {
        const std::string key = r.str();
        const uint32_t type = r.get<uint32_t>();
        skip_gguf_value(r, type, key == "general.alignment" ? &alignment : nullptr);
    }
    for (uint64_t i = 0; i < n_tensors && r.ok; i++) {
        TensorInfo t;
        t.name = r.str();
        const uint32_t nd = r.get<uint32_t>();
        if (nd > 4) { r.ok = false; break; }
        t.ndim = (int)nd;
        for (uint32_t d = 0; d < nd; d++) t.shape[d] = r.get<uint64_t>();
        const uint32_t type = r.get<uint32_t>();
        t.dtype = (type == MF_F32 || type == MF_F16 || type == MF_Q8_0) ? (int)type : -1;
        t.begin = r.get<uint64_t>();
        if (t.elements() == UINT64_MAX) { r.ok = false; break; }      // dimensions whose product overflows
        t.nbytes = bytes_of(t.dtype, t.elements());
        f->tensors.push_back(t);
    }
    if (!r.ok || alignment == 0) { fprintf(stderr, "[Loader] %s: truncated or malformed GGUF header\n", path.c_str()); f->tensors.clear(); munmap(m.p, m.size); return false; }
    m.data_off = (r.off + alignment - 1) / alignment * alignment;
    for (const TensorInfo &t : f->tensors)
        if (!range_inside(m.data_off, t.begin, t.nbytes, m.size)) {
            fprintf(stderr, "[Loader] %s: tensor %s lies outside the file\n", path.c_str(), t.name.c_str());
            f->tensors.clear(); munmap(m.p, m.size);
            return false;
        }
    f->maps.push_back(m);
    f->gguf = true;
    return true;
}

const TensorInfo *find(ModelFile *f, const char *name)
{
    auto it = f->index.find(name);
    return it == f->index.end() ? nullptr : &f->tensors[it->second];
}

const uint8_t *bytes(ModelFile *f, const TensorInfo *t) { const Mapping &m = f->maps[t->shard]; return (const uint8_t *)m.p + m.data_off + t->begin; }

float half_bits_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h >> 15) << 31, exp = (h >> 10) & 31, man = h & 1023;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) bits = sign;
        else { int e = -1; uint32_t m = man; do { e++; m <<= 1; } while (!(m & 1024)); bits = sign | ((uint32_t)(112 - e) << 23) | ((m & 1023) << 13); }
    } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
    else bits = sign | ((exp + 112) << 23) | (man << 13);
    float v;
    memcpy(&v, &bits, 4);
    return v;
}

void widen(const uint8_t *src, int dtype, uint64_t n, float *dst)
{
    if (dtype == MF_F32) memcpy(dst, src, n * 4);
    else if (dtype == MF_F16) { for (uint64_t i = 0; i < n; i++) { uint16_t h; memcpy(&h, src + 2 * i, 2); dst[i] = half_bits_to_float(h); } }
    else if (dtype == MF_BF16) { for (uint64_t i = 0; i < n; i++) { uint16_t h; memcpy(&h, src + 2 * i, 2); const uint32_t b = (uint32_t)h << 16; memcpy(&dst[i], &b, 4); } }
    else if (dtype == MF_Q8_0) {
        for (uint64_t b = 0; b * 32 < n; b++) {
            const uint8_t *blk = src + b * 34;
            uint16_t h;
            memcpy(&h, blk, 2);
            const float scale = half_bits_to_float(h);
            const uint64_t cnt = std::min<uint64_t>(32, n - b * 32);
            for (uint64_t i = 0; i < cnt; i++) dst[b * 32 + i] = (float)(int8_t)blk[2 + i] * scale;
        }
    }
}

// ---------------------------------------------------------------- device side of model_file_load_wmat

__global__ __launch_bounds__(256) void k_widen16(const uint16_t *__restrict__ src, float *__restrict__ dst, size_t n, int bf16)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const uint16_t h = src[i];
    dst[i] = bf16 ? __uint_as_float((uint32_t)h << 16) : (float)__builtin_bit_cast(half_t, h);
}

// ---------------------------------------------------------------- model description

struct OwnedRef {
    SFTModelRef ref;
    std::vector<float *> owned;
    std::vector<LayerWeightRef> layers;
    std::vector<float> thetas;
};
std::map<SFTModelRef *, OwnedRef *> g_refs;      // descriptions handed out by model_ref_load

std::string layer_name(bool gguf, int L, const char *hf, const char *gg)
{
    char buf[256];
    if (gguf) snprintf(buf, sizeof buf, "blk.%d.%s.weight", L, gg);
    else snprintf(buf, sizeof buf, "model.layers.%d.%s.weight", L, hf);
    return buf;
}

}  // namespace

extern "C" {

ModelFile *model_file_open(const char *path)
{
    struct stat st;
    if (!path || stat(path, &st) != 0) { fprintf(stderr, "[Loader] cannot access %s\n", path ? path : "(null)"); return nullptr; }
    ModelFile *f = new ModelFile();
    bool ok = true;
    if (S_ISDIR(st.st_mode)) {
        std::vector<std::string> shards;
        if (DIR *d = opendir(path)) {
            while (struct dirent *e = readdir(d)) {
                const std::string n = e->d_name;
                if (n.size() > 12 && n.compare(n.size() - 12, 12, ".safetensors") == 0) shards.push_back(std::string(path) + "/" + n);
            }
            closedir(d);
        }
        std::sort(shards.begin(), shards.end());
        if (shards.empty()) { fprintf(stderr, "[Loader] no .safetensors files in %s\n", path); ok = false; }
        for (const std::string &s : shards) ok = ok && open_safetensors_shard(s, f);
    } else {
        uint32_t magic = 0;
        if (FILE *fp = fopen(path, "rb")) { if (fread(&magic, 4, 1, fp) != 1) magic = 0; fclose(fp); }
        ok = magic == 0x46554747u ? open_gguf(path, f) : open_safetensors_shard(path, f);
    }
    if (!ok) { model_file_close(f); return nullptr; }
    for (size_t i = 0; i < f->tensors.size(); i++) f->index.emplace(f->tensors[i].name, (int)i);   // first of equal names wins
    return f;
}

void model_file_close(ModelFile *f)
{
    if (!f) return;
    for (Mapping &m : f->maps) if (m.p) munmap(m.p, m.size);
    delete f;
}

int model_file_is_gguf(ModelFile *f) { return f->gguf ? 1 : 0; }
int model_file_count(ModelFile *f) { return (int)f->tensors.size(); }
const char *model_file_name(ModelFile *f, int i) { return i >= 0 && i < (int)f->tensors.size() ? f->tensors[i].name.c_str() : nullptr; }

int model_file_find(ModelFile *f, const char *name, int *dtype, int *ndim, uint64_t shape[4])
{
    const TensorInfo *t = find(f, name);
    if (!t) return 0;
    if (dtype) *dtype = t->dtype;
    if (ndim) *ndim = t->ndim;
    if (shape) memcpy(shape, t->shape, sizeof t->shape);
    return 1;
}

int model_file_matrix_shape(ModelFile *f, const char *name, int *rows, int *cols)
{
    const TensorInfo *t = find(f, name);
    if (!t || t->ndim < 1 || t->ndim > 2) return 0;
    uint64_t r, c;
    if (t->ndim == 1) { r = 1; c = t->shape[0]; }
    else if (f->gguf) { c = t->shape[0]; r = t->shape[1]; }
    else { r = t->shape[0]; c = t->shape[1]; }
    if (r > 0x7fffffff || c > 0x7fffffff) return 0;
    *rows = (int)r; *cols = (int)c;
    return 1;
}

const void *model_file_data(ModelFile *f, const char *name, size_t *nbytes)
{
    const TensorInfo *t = find(f, name);
    if (!t) return nullptr;
    if (nbytes) *nbytes = t->nbytes;
    return bytes(f, t);
}

float *model_file_load_f32(ModelFile *f, const char *name, size_t *n_elements)
{
    if (n_elements) *n_elements = 0;
    const TensorInfo *t = find(f, name);
    if (!t) { fprintf(stderr, "[Loader] tensor not found: %s\n", name); return nullptr; }
    if (t->dtype < 0) { fprintf(stderr, "[Loader] unsupported element type of %s\n", name); return nullptr; }
    const uint64_t n = t->elements();
    float *out = (float *)malloc(std::max<uint64_t>(n, 1) * sizeof(float));
    if (!out) { fprintf(stderr, "[Loader] out of memory for %s (%llu elements)\n", name, (unsigned long long)n); return nullptr; }
    widen(bytes(f, t), t->dtype, n, out);
    if (n_elements) *n_elements = n;
    return out;
}

WMat *model_file_load_wmat(ModelFile *f, const char *name, int use_fp16)
{
    const TensorInfo *t = find(f, name);
    int rows = 0, cols = 0;
    if (!t || t->dtype < 0 || !model_file_matrix_shape(f, name, &rows, &cols)) {
        fprintf(stderr, "[Loader] %s: absent, of unsupported type or not a matrix\n", name);
        return nullptr;
    }
    if (!use_fp16 && cols % 32) { fprintf(stderr, "[Loader] %s: %d columns are not a multiple of 32 (Q8_0)\n", name, cols); return nullptr; }
    if (!initialized()) { fprintf(stderr, "[Loader] model_file_load_wmat before fast_metal_init\n"); return nullptr; }
    WMat *w = (WMat *)calloc(1, sizeof(WMat));
    w->rows = rows; w->cols = cols; w->nb = use_fp16 ? 0 : cols / 32;
    const size_t n = (size_t)rows * cols;
    MetalBuf *raw = metal_buf_from_data(bytes(f, t), t->nbytes);
    const bool as_is = (use_fp16 && t->dtype == MF_F16) || (!use_fp16 && t->dtype == MF_Q8_0);
    if (as_is) { w->mbuf = raw; return w; }
    w->mbuf = metal_buf_create(use_fp16 ? n * 2 : (size_t)rows * w->nb * 34);
    if (use_fp16 && t->dtype == MF_Q8_0) {
        hip_enqueue_q8_to_f16(raw, w->mbuf, rows, cols);
    } else {
        MetalBuf *wide = raw;
        if (t->dtype != MF_F32) {
            wide = metal_buf_create(n * 4);
            if (t->dtype == MF_Q8_0) hip_enqueue_q8_dequant(raw, wide, rows, cols);
            else hipLaunchKernelGGL(k_widen16, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream(), dptr_as<uint16_t>(raw),
                                    dptr_as<float>(wide), n, t->dtype == MF_BF16 ? 1 : 0);
        }
        if (use_fp16) hip_enqueue_f32_to_f16(wide, w->mbuf, n);
        else hip_enqueue_q8_quantize(wide, w->mbuf, rows, cols);
        if (wide != raw) metal_buf_free(wide);
    }
    metal_buf_free(raw);                                      // synchronises the stream first
    return w;
}

SFTModelRef *model_ref_load(const char *path, ModelType model_type)
{
    ModelFile *f = model_file_open(path);
    if (!f) return nullptr;
    const bool gg = f->gguf;
    if (gg && model_type == MODEL_GEMMA3) { fprintf(stderr, "[Loader] Gemma3 is read from safetensors only\n"); model_file_close(f); return nullptr; }
    OwnedRef *o = new OwnedRef();
    bool ok = true;
    // fp32 copy of a tensor with an expected element count (0: any); Gemma3 norm weights get + 1.0
    auto load = [&](const std::string &name, size_t expect, bool norm, bool required = true) -> float * {
        if (!find(f, name.c_str())) { if (required) { fprintf(stderr, "[Loader] tensor '%s' not found\n", name.c_str()); ok = false; } return nullptr; }
        size_t n = 0;
        float *d = model_file_load_f32(f, name.c_str(), &n);
        if (!d || (expect && n != expect)) {
            fprintf(stderr, "[Loader] size mismatch for '%s': file=%zu, model=%zu\n", name.c_str(), n, expect);
            free(d); ok = false;
            return nullptr;
        }
        if (norm && model_type == MODEL_GEMMA3) for (size_t i = 0; i < n; i++) d[i] += 1.0f;
        o->owned.push_back(d);
        return d;
    };
    const char *emb_name = gg ? "token_embd.weight" : "model.embed_tokens.weight";
    int V = 0, D = 0, NL = 0;
    if (!model_file_matrix_shape(f, emb_name, &V, &D)) { fprintf(stderr, "[Loader] tensor '%s' not found\n", emb_name); ok = false; }
    while (ok && find(f, layer_name(gg, NL, "self_attn.q_proj", "attn_q").c_str())) NL++;
    int qd = 0, kd = 0, IS = 0, hd = 0, one = 0, c = 0;
    if (ok && NL > 0) {
        ok = model_file_matrix_shape(f, layer_name(gg, 0, "self_attn.q_proj", "attn_q").c_str(), &qd, &c) && c == D &&
             model_file_matrix_shape(f, layer_name(gg, 0, "self_attn.k_proj", "attn_k").c_str(), &kd, &c) && c == D &&
             model_file_matrix_shape(f, layer_name(gg, 0, "mlp.gate_proj", "ffn_gate").c_str(), &IS, &c) && c == D &&
             model_file_matrix_shape(f, layer_name(gg, 0, "self_attn.q_norm", "attn_q_norm").c_str(), &one, &hd) && hd > 0 &&
             qd % hd == 0 && kd % hd == 0;
        if (!ok) fprintf(stderr, "[Loader] layer 0 tensors missing or inconsistent with d_model %d\n", D);
    } else if (ok) { fprintf(stderr, "[Loader] no transformer layers found\n"); ok = false; }
    if (ok) {
        o->layers.resize(NL);
        o->thetas.resize(NL);
        const bool gemma = model_type == MODEL_GEMMA3;
        for (int L = 0; L < NL && ok; L++) {
            LayerWeightRef &r = o->layers[L];
            auto mat = [&](const char *hf, const char *g, int rows, int cols) { return WeightRef{load(layer_name(gg, L, hf, g), (size_t)rows * cols, false), rows, cols}; };
            r.input_norm_g = load(layer_name(gg, L, "input_layernorm", "attn_norm"), D, true);
            r.q_proj = mat("self_attn.q_proj", "attn_q", qd, D);
            r.k_proj = mat("self_attn.k_proj", "attn_k", kd, D);
            r.v_proj = mat("self_attn.v_proj", "attn_v", kd, D);
            r.q_norm_g = load(layer_name(gg, L, "self_attn.q_norm", "attn_q_norm"), hd, true);
            r.k_norm_g = load(layer_name(gg, L, "self_attn.k_norm", "attn_k_norm"), hd, true);
            r.o_proj = mat("self_attn.o_proj", "attn_output", D, qd);
            r.post_attn_norm_g = load(layer_name(gg, L, "post_attention_layernorm", "ffn_norm"), D, true);
            r.pre_ff_norm_g = gemma ? load(layer_name(gg, L, "pre_feedforward_layernorm", ""), D, true) : nullptr;
            r.gate_proj = mat("mlp.gate_proj", "ffn_gate", IS, D);
            r.up_proj = mat("mlp.up_proj", "ffn_up", IS, D);
            r.down_proj = mat("mlp.down_proj", "ffn_down", D, IS);
            r.post_ff_norm_g = gemma ? load(layer_name(gg, L, "post_feedforward_layernorm", ""), D, true) : nullptr;
            r.d_model = D; r.head_dim = hd;
            o->thetas[L] = gemma ? ((L % 6) != 0 ? 1e4f : 1e6f) : 1e6f;     // src/nn/fast_sft.c:308-313; qwen3_4b_config
        }
    }
    SFTModelRef &m = o->ref;
    memset(&m, 0, sizeof m);
    if (ok) {
        m.model_type = model_type;
        m.n_layers = NL; m.d_model = D; m.n_q_heads = qd / hd; m.n_kv_heads = kd / hd; m.head_dim = hd;
        m.intermediate_size = IS; m.vocab_size = V;
        m.rope_thetas = o->thetas.data();
        m.layers = o->layers.data();
        m.token_emb = load(emb_name, (size_t)V * D, false);
        m.final_norm_g = load(gg ? "output_norm.weight" : "model.norm.weight", D, true);
        // Gemma3 ties the LM head to the embedding; Qwen3 files may (src/nn/qwen3.c:264-270, 363-367)
        const float *head = model_type == MODEL_GEMMA3 ? nullptr : load(gg ? "output.weight" : "lm_head.weight", (size_t)V * D, false, false);
        m.lm_head = head ? head : m.token_emb;
        m.lora_init = nullptr;
    }
    model_file_close(f);
    if (!ok) { for (float *p : o->owned) free(p); delete o; return nullptr; }
    g_refs[&o->ref] = o;
    return &o->ref;
}

void model_ref_free(SFTModelRef *m)
{
    auto it = g_refs.find(m);
    if (it == g_refs.end()) return;
    OwnedRef *o = it->second;
    g_refs.erase(it);
    for (float *p : o->owned) free(p);
    delete o;
}

}  // extern "C"
