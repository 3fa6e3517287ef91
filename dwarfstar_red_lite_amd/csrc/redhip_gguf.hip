// GGUF side of the resident MoE layers: finds the router, shared-expert and routed-expert tensors of every layer in a
// GGUF v2 / v3 file and uploads them through the redhip_moe_load_* entry points. Host code only.
//
// Reference behaviour: the tensor directory walk and the expert byte ranges of native/redlite_native_gguf.c:196-440
// (blk.N.ffn_{gate,up,down}_exps.weight are expert-major and contiguous, one expert = dims[0] x dims[1] weights) and
// the per-layer tensor names and shapes the engine expects, native/redlite_native_engine.c:170-179.
#include <errno.h>
#include <fcntl.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>
#include <sys/stat.h>
#include <unistd.h>

#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/redhip_moe.h"
#include "redhip_internal.h"

namespace {

using namespace redhip;

thread_local char g_gguf_error[512];
void gguf_err(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_gguf_error, sizeof(g_gguf_error), fmt, ap);
    va_end(ap);
}

struct Tensor {
    uint32_t type = 0, n_dims = 0;
    uint64_t dims[4] = {1, 1, 1, 1};
    uint64_t offset = 0;          // absolute file offset of the data
    uint64_t bytes = 0;           // 0 when the type is not one this library sizes
};

struct File {
    int fd = -1;
    uint64_t size = 0, pos = 0;
    std::vector<uint8_t> buf;     // window of the file used while parsing the directory
    uint64_t buf_start = 0;
    ~File() { if (fd >= 0) close(fd); }

    bool read(void *dst, uint64_t n) {
        if (pos + n > size) return false;
        if (pos < buf_start || pos + n > buf_start + buf.size()) {
            const uint64_t want = n > (1u << 20) ? n : (1u << 20), len = pos + want > size ? size - pos : want;
            buf.resize((size_t)len);
            uint64_t got = 0;
            while (got < len) {
                const ssize_t r = pread(fd, buf.data() + got, (size_t)(len - got), (off_t)(pos + got));
                if (r <= 0) return false;
                got += (uint64_t)r;
            }
            buf_start = pos;
        }
        memcpy(dst, buf.data() + (pos - buf_start), (size_t)n);
        pos += n;
        return true;
    }
    template <class T> bool get(T *v) { return read(v, sizeof(T)); }
    bool skip(uint64_t n) { if (pos + n > size) return false; pos += n; return true; }
    bool str(std::string *s) {
        uint64_t n = 0;
        if (!get(&n) || n > (1u << 20)) return false;
        s->resize((size_t)n);
        return n == 0 || read(&(*s)[0], n);
    }
};

// size in bytes of a scalar GGUF metadata value type, 0 for strings / arrays
uint64_t scalar_size(uint32_t t) {
    switch (t) {
        case 0: case 1: case 7: return 1;
        case 2: case 3: return 2;
        case 4: case 5: case 6: return 4;
        case 10: case 11: case 12: return 8;
        default: return 0;
    }
}

bool skip_value(File &f, uint32_t type, int depth = 0) {
    if (const uint64_t n = scalar_size(type)) return f.skip(n);
    if (type == 8) { std::string s; return f.str(&s); }
    if (type == 9 && depth < 2) {
        uint32_t et = 0;
        uint64_t count = 0;
        if (!f.get(&et) || !f.get(&count)) return false;
        if (const uint64_t n = scalar_size(et)) return count <= f.size / n && f.skip(n * count);
        for (uint64_t i = 0; i < count; ++i) if (!skip_value(f, et, depth + 1)) return false;
        return true;
    }
    return false;
}

struct Directory {
    std::unordered_map<std::string, Tensor> tensors;
    std::unordered_map<std::string, uint64_t> ints;      // integer metadata values by key
};

uint64_t tensor_bytes(uint32_t type, const uint64_t *dims, uint32_t n_dims) {
    uint64_t rows = 1;
    for (uint32_t i = 1; i < n_dims; ++i) rows *= dims[i];
    if (type == T_F32) return dims[0] * rows * 4u;
    if (!pool_quant_supported(type) || dims[0] % 256u) return 0;
    return rows * pool_row_bytes(type, (uint32_t)dims[0]);
}

bool parse(const char *path, File &f, Directory &d) {
    f.fd = open(path, O_RDONLY);
    struct stat st;
    if (f.fd < 0 || fstat(f.fd, &st) != 0) { gguf_err("open %s failed: %s", path, strerror(errno)); return false; }
    f.size = (uint64_t)st.st_size;
    char magic[4];
    uint32_t version = 0;
    uint64_t n_tensor = 0, n_kv = 0;
    if (!f.read(magic, 4) || memcmp(magic, "GGUF", 4) != 0 || !f.get(&version) || (version != 2u && version != 3u) ||
        !f.get(&n_tensor) || !f.get(&n_kv) || n_tensor > f.size / 24u) {
        gguf_err("invalid or unsupported GGUF header in %s", path);
        return false;
    }
    uint64_t alignment = 32;
    for (uint64_t i = 0; i < n_kv; ++i) {
        std::string key;
        uint32_t type = 0;
        if (!f.str(&key) || !f.get(&type)) { gguf_err("failed to parse GGUF metadata"); return false; }
        if (type == 4 || type == 5) { uint32_t v = 0; if (!f.get(&v)) return false; d.ints[key] = v; }
        else if (type == 10 || type == 11) { uint64_t v = 0; if (!f.get(&v)) return false; d.ints[key] = v; }
        else if (!skip_value(f, type)) { gguf_err("failed to parse GGUF metadata value of %s", key.c_str()); return false; }
    }
    if (d.ints.count("general.alignment") && d.ints["general.alignment"]) alignment = d.ints["general.alignment"];
    std::vector<std::pair<std::string, Tensor>> list;
    list.reserve((size_t)n_tensor);
    for (uint64_t i = 0; i < n_tensor; ++i) {
        std::string name;
        Tensor t;
        if (!f.str(&name) || !f.get(&t.n_dims) || t.n_dims == 0 || t.n_dims > 4) { gguf_err("failed to parse GGUF tensor directory"); return false; }
        for (uint32_t k = 0; k < t.n_dims; ++k) if (!f.get(&t.dims[k]) || !t.dims[k]) { gguf_err("failed to parse GGUF tensor directory"); return false; }
        if (!f.get(&t.type) || !f.get(&t.offset)) { gguf_err("failed to parse GGUF tensor directory"); return false; }
        t.bytes = tensor_bytes(t.type, t.dims, t.n_dims);
        list.emplace_back(std::move(name), t);
    }
    const uint64_t data_start = (f.pos + alignment - 1u) / alignment * alignment;
    for (auto &kv : list) {
        kv.second.offset += data_start;
        if (kv.second.bytes && kv.second.offset + kv.second.bytes > f.size) { gguf_err("tensor %s reaches beyond the end of the file", kv.first.c_str()); return false; }
        d.tensors[kv.first] = kv.second;
    }
    return true;
}

const Tensor *find(const Directory &d, uint32_t layer, const char *suffix) {
    char name[96];
    snprintf(name, sizeof(name), "blk.%u.%s", layer, suffix);
    const auto it = d.tensors.find(name);
    return it == d.tensors.end() ? nullptr : &it->second;
}

bool read_tensor(File &f, const Tensor &t, std::vector<uint8_t> &out) {
    out.resize((size_t)t.bytes);
    uint64_t got = 0;
    while (got < t.bytes) {
        const ssize_t r = pread(f.fd, out.data() + got, (size_t)(t.bytes - got), (off_t)(t.offset + got));
        if (r <= 0) { gguf_err("short read of a tensor: %s", strerror(errno)); return false; }
        got += (uint64_t)r;
    }
    return true;
}

// the seven MoE tensors of a layer, with their shapes checked against each other
struct LayerTensors {
    const Tensor *router, *gate_inp, *sh_gate, *sh_up, *sh_down, *gate, *up, *down;
};

bool layer_tensors(const Directory &d, uint32_t layer, LayerTensors &t) {
    t.router = find(d, layer, "ffn_gate_inp.weight");
    t.gate_inp = find(d, layer, "ffn_gate_inp_shexp.weight");
    t.sh_gate = find(d, layer, "ffn_gate_shexp.weight");
    t.sh_up = find(d, layer, "ffn_up_shexp.weight");
    t.sh_down = find(d, layer, "ffn_down_shexp.weight");
    t.gate = find(d, layer, "ffn_gate_exps.weight");
    t.up = find(d, layer, "ffn_up_exps.weight");
    t.down = find(d, layer, "ffn_down_exps.weight");
    if (!t.router || !t.gate_inp || !t.sh_gate || !t.sh_up || !t.sh_down || !t.gate || !t.up || !t.down) {
        gguf_err("layer %u lacks one of the MoE tensors (ffn_gate_inp, ffn_gate_inp_shexp, ffn_{gate,up,down}_shexp, ffn_{gate,up,down}_exps)", layer);
        return false;
    }
    const uint64_t H = t.router->dims[0], E = t.router->dims[1], F = t.gate->dims[1];
    const bool ok = t.router->n_dims == 2 && t.gate->n_dims == 3 && t.up->n_dims == 3 && t.down->n_dims == 3 &&
                    t.gate->dims[0] == H && t.gate->dims[2] == E && t.up->dims[0] == H && t.up->dims[1] == F && t.up->dims[2] == E &&
                    t.down->dims[0] == F && t.down->dims[1] == H && t.down->dims[2] == E && t.gate->type == t.up->type &&
                    t.sh_gate->dims[0] == H && t.sh_up->dims[0] == H && t.sh_gate->dims[1] == F && t.sh_up->dims[1] == F &&
                    t.sh_down->dims[0] == F && t.sh_down->dims[1] == H && t.sh_gate->type == t.sh_up->type &&
                    t.gate_inp->type == T_F32 && t.gate_inp->dims[0] == H;
    if (!ok) gguf_err("layer %u: MoE tensor shapes or types do not fit together (the shared expert must have the routed experts' width)", layer);
    return ok;
}

}  // namespace

extern "C" {

const char *redhip_gguf_last_error(void) { return g_gguf_error[0] ? g_gguf_error : "unknown redhip GGUF error"; }

int redhip_gguf_moe_config(const char *path, uint32_t first_layer, redhip_moe_config *out) {
    g_gguf_error[0] = '\0';
    if (!path || !out) { gguf_err("invalid GGUF configuration request"); return 0; }
    File f;
    Directory d;
    if (!parse(path, f, d)) return 0;
    LayerTensors t;
    if (!layer_tensors(d, first_layer, t)) return 0;
    memset(out, 0, sizeof(*out));
    out->hidden = (uint32_t)t.router->dims[0];
    out->n_expert = (uint32_t)t.router->dims[1];
    out->ffn = (uint32_t)t.gate->dims[1];
    out->router_type = t.router->type;
    out->expert_type_word = t.gate->type == t.down->type ? t.gate->type : (t.gate->type | (t.down->type << 8));
    out->shared_type_word = t.sh_gate->type == t.sh_down->type ? t.sh_gate->type : (t.sh_gate->type | (t.sh_down->type << 8));
    for (const auto &kv : d.ints) {
        const std::string &k = kv.first;
        if (k.size() > 18 && k.compare(k.size() - 18, 18, ".expert_used_count") == 0) out->top_k = (uint32_t)kv.second;
    }
    // the run of layers from first_layer that share its shapes and types: a file whose layers differ in their expert format (the
    // reference's target file holds IQ2_XS in its first and last layers and IQ1_M between) is walked as one run per format
    uint32_t n = 0;
    LayerTensors probe;
    while (find(d, first_layer + n, "ffn_gate_exps.weight") && layer_tensors(d, first_layer + n, probe) &&
           probe.gate->type == t.gate->type && probe.down->type == t.down->type && probe.sh_gate->type == t.sh_gate->type &&
           probe.sh_down->type == t.sh_down->type && probe.router->type == t.router->type && probe.router->dims[0] == t.router->dims[0] &&
           probe.router->dims[1] == t.router->dims[1] && probe.gate->dims[1] == t.gate->dims[1]) ++n;
    g_gguf_error[0] = '\0';
    out->n_layer = n;
    out->max_tokens = 1;
    if (!out->top_k) { gguf_err("no <architecture>.expert_used_count in the GGUF metadata"); return 0; }
    return 1;
}

int redhip_gguf_expert_layout(const char *path, uint32_t expected_experts, uint32_t layer, uint32_t expert, redhip_gguf_expert_layout_t *out) {
    g_gguf_error[0] = '\0';
    if (!path || !out || !expected_experts || expert >= expected_experts) { gguf_err("invalid expert layout request"); return 0; }
    File f;
    Directory d;
    if (!parse(path, f, d)) return 0;
    const Tensor *t[3] = {find(d, layer, "ffn_gate_exps.weight"), find(d, layer, "ffn_up_exps.weight"), find(d, layer, "ffn_down_exps.weight")};
    if (!t[0] || !t[1] || !t[2]) { gguf_err("layer %u does not contain routed gate/up/down tensors", layer); return 0; }
    uint64_t per[3];
    for (int k = 0; k < 3; ++k) {
        // the expert index is the slowest dimension, so one expert is a contiguous range of the tensor
        if (t[k]->n_dims < 2 || t[k]->dims[t[k]->n_dims - 1] != expected_experts || !t[k]->bytes || t[k]->bytes % expected_experts) {
            gguf_err("layer %u: a routed tensor is not sliceable by expert (expert count %u is not its last dimension, or its type is not sized here)", layer, expected_experts);
            return 0;
        }
        per[k] = t[k]->bytes / expected_experts;
    }
    if (t[0]->type != t[1]->type) { gguf_err("layer %u: routed gate and up tensors must share one quantisation type", layer); return 0; }
    memset(out, 0, sizeof(*out));
    out->layer = layer;
    out->expert = expert;
    out->ggml_type = t[0]->type;
    out->down_type = t[2]->type;
    out->gate_offset = t[0]->offset + expert * per[0];
    out->gate_bytes = per[0];
    out->up_offset = t[1]->offset + expert * per[1];
    out->up_bytes = per[1];
    out->down_offset = t[2]->offset + expert * per[2];
    out->down_bytes = per[2];
    out->total_bytes = per[0] + per[1] + per[2];
    return 1;
}

int redhip_moe_load_gguf(redhip_moe_t moe, const char *path, uint32_t first_layer, uint32_t n_layer, const redhip_moe_config *cfg) {
    g_gguf_error[0] = '\0';
    if (!moe || !path || !cfg || !n_layer || n_layer > cfg->n_layer) { gguf_err("invalid GGUF load request"); return 0; }
    File f;
    Directory d;
    if (!parse(path, f, d)) return 0;
    const uint32_t gu = cfg->expert_type_word & 255u, dn = (cfg->expert_type_word >> 8) ? (cfg->expert_type_word >> 8) : gu;
    const uint32_t sgu = cfg->shared_type_word & 255u, sdn = (cfg->shared_type_word >> 8) ? (cfg->shared_type_word >> 8) : sgu;
    std::vector<uint8_t> a, b, c, gi;
    for (uint32_t l = 0; l < n_layer; ++l) {
        LayerTensors t;
        if (!layer_tensors(d, first_layer + l, t)) return 0;
        if (t.router->dims[0] != cfg->hidden || t.router->dims[1] != cfg->n_expert || t.gate->dims[1] != cfg->ffn || t.router->type != cfg->router_type ||
            t.gate->type != gu || t.down->type != dn || t.sh_gate->type != sgu || t.sh_down->type != sdn || !t.router->bytes || !t.gate->bytes ||
            !t.down->bytes || !t.sh_gate->bytes || !t.sh_down->bytes) {
            gguf_err("layer %u of %s does not match the MoE configuration (shape or quantisation types)", first_layer + l, path);
            return 0;
        }
        if (!read_tensor(f, *t.router, a)) return 0;
        if (!redhip_moe_load_router(moe, l, a.data(), a.size())) { gguf_err("router upload: %s", redhip_moe_last_error()); return 0; }
        if (!read_tensor(f, *t.gate_inp, gi) || !read_tensor(f, *t.sh_gate, a) || !read_tensor(f, *t.sh_up, b) || !read_tensor(f, *t.sh_down, c)) return 0;
        if (!redhip_moe_load_shared(moe, l, reinterpret_cast<const float *>(gi.data()), a.data(), a.size(), b.data(), b.size(), c.data(), c.size())) {
            gguf_err("shared expert upload: %s", redhip_moe_last_error());
            return 0;
        }
        if (!read_tensor(f, *t.gate, a) || !read_tensor(f, *t.up, b) || !read_tensor(f, *t.down, c)) return 0;
        if (!redhip_moe_load_experts(moe, l, 0u, cfg->n_expert, a.data(), b.data(), c.data())) { gguf_err("expert upload: %s", redhip_moe_last_error()); return 0; }
    }
    return 1;
}

}  // extern "C"
