// Wire-format shim of the worker contract: safetensors {"data"} in, safetensors
// {"data"} out, one expert per call, expert ids as "{model}/l{L}-e{E}".
//
// Follows EKInstanceGate::forward (ek-computation/src/worker/core.rs:47-74): the
// request tensor is read with SafeTensors::deserialize + tensor("data") (:52-53),
// the expert is taken from sequences[0].experts[0] (:55-57), the result is written
// with TchTensor::serialize = write_safetensors(&[("data", ..)])
// (backend/torch/mod.rs:115-117).  Id codec: ExpertKey::from_expert_id /
// as_object_key (ek-db/src/safetensor/mod.rs:57-90).
//
// ek_worker_forward_batch is the micro-batcher: the controller fires one such call
// per expert concurrently (controller/executor.rs:141-195); a worker that collects
// them hands all of them over at once and they run as ONE grouped launch.
#include "../../include/ek_hip.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

namespace ekw {

struct DtypeName { const char *name; int32_t dtype; int32_t size; };
// names of safetensors::Dtype that map onto ek_dtype (backend/torch/tch_safetensors.rs:12-46)
static const DtypeName kDtypes[] = {{"BF16", EK_BF16, 2}, {"F16", EK_F16, 2}, {"F32", EK_F32, 4},
                                    {"I8", EK_I8, 1},     {"F8_E4M3", EK_F8E4M3, 1}};

// ---- a JSON reader just big enough for a safetensors header -------------------
struct Cursor {
    const char *p, *end;
    void ws() { while (p < end && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) ++p; }
    bool eat(char c) { ws(); if (p < end && *p == c) { ++p; return true; } return false; }
    bool string(std::string &out)
    {
        ws();
        if (p >= end || *p != '"') return false;
        ++p;
        out.clear();
        while (p < end && *p != '"') {
            if (*p == '\\') {
                if (++p >= end) return false;
                switch (*p) {
                case 'n': out.push_back('\n'); break;
                case 't': out.push_back('\t'); break;
                case 'u': if (end - p < 5) return false; out.push_back('?'); p += 4; break;
                default: out.push_back(*p);
                }
                ++p;
            } else {
                out.push_back(*p++);
            }
        }
        if (p >= end) return false;
        ++p;
        return true;
    }
    bool integer(int64_t &v)
    {
        ws();
        const char *s = p;
        if (p < end && *p == '-') ++p;
        if (p >= end || *p < '0' || *p > '9') { p = s; return false; }
        int64_t acc = 0;
        while (p < end && *p >= '0' && *p <= '9') {
            if (acc > (INT64_MAX - 9) / 10) return false;
            acc = acc * 10 + (*p++ - '0');
        }
        v = *s == '-' ? -acc : acc;
        return true;
    }
    // skips any JSON value.  Wire bytes are untrusted: nesting beyond kMaxDepth is refused (the
    // recursion would otherwise be as deep as the header is long; a safetensors header nests
    // three levels, and the reference's parser rejects a __metadata__ that is not flat)
    static constexpr int kMaxDepth = 32;
    bool skip(int depth = 0)
    {
        if (depth > kMaxDepth) return false;
        ws();
        if (p >= end) return false;
        if (*p == '"') { std::string t; return string(t); }
        if (*p == '{' || *p == '[') {
            const char open = *p, close = open == '{' ? '}' : ']';
            ++p;
            if (eat(close)) return true;
            while (true) {
                if (open == '{') { std::string k; if (!string(k) || !eat(':')) return false; }
                if (!skip(depth + 1)) return false;
                if (eat(',')) continue;
                return eat(close);
            }
        }
        while (p < end && *p != ',' && *p != '}' && *p != ']') ++p;   // number / true / false / null
        return true;
    }
};

struct Entry {
    std::string dtype;
    std::vector<int64_t> shape;
    int64_t begin = -1, end = -1;
};

static bool parse_entry(Cursor &c, Entry &e)
{
    if (!c.eat('{')) return false;
    if (c.eat('}')) return true;
    while (true) {
        std::string key;
        if (!c.string(key) || !c.eat(':')) return false;
        if (key == "dtype") {
            if (!c.string(e.dtype)) return false;
        } else if (key == "shape") {
            if (!c.eat('[')) return false;
            if (!c.eat(']')) {
                while (true) {
                    int64_t v;
                    if (!c.integer(v) || v < 0) return false;
                    e.shape.push_back(v);
                    if (c.eat(',')) continue;
                    if (!c.eat(']')) return false;
                    break;
                }
            }
        } else if (key == "data_offsets") {
            if (!c.eat('[') || !c.integer(e.begin) || !c.eat(',') || !c.integer(e.end) || !c.eat(']')) return false;
        } else if (!c.skip()) {
            return false;
        }
        if (c.eat(',')) continue;
        return c.eat('}');
    }
}

}  // namespace ekw

namespace ek { void set_last_error(const char *msg); }   // the thread's ek_last_error() text

static ek_status wire_fail(ek_status st, const std::string &msg)
{
    ek::set_last_error(msg.c_str());
    return st;
}

extern "C" {

ek_status ek_expert_id_parse(const char *id, int32_t *layer, int32_t *expert)
{
    // id.split("/l") must give exactly two parts, the second split("-e") exactly two,
    // both numeric (ek-db/src/safetensor/mod.rs:57-73)
    if (!id || !layer || !expert) return wire_fail(EK_INVALID_INPUT, "NULL argument");
    const std::string s(id);
    const size_t a = s.find("/l");
    if (a == std::string::npos || s.find("/l", a + 2) != std::string::npos)
        return wire_fail(EK_INVALID_INPUT, "invalid expert id: " + s);
    const std::string rest = s.substr(a + 2);
    const size_t b = rest.find("-e");
    if (b == std::string::npos || rest.find("-e", b + 2) != std::string::npos)
        return wire_fail(EK_INVALID_INPUT, "invalid expert id: " + s);
    const std::string ls = rest.substr(0, b), es = rest.substr(b + 2);
    auto numeric = [](const std::string &t) {
        if (t.empty() || t.size() > 9) return false;
        for (char ch : t) if (ch < '0' || ch > '9') return false;
        return true;
    };
    // Rust's usize parse also accepts a leading '+'
    auto strip = [](const std::string &t) { return !t.empty() && t[0] == '+' ? t.substr(1) : t; };
    if (!numeric(strip(ls)) || !numeric(strip(es))) return wire_fail(EK_INVALID_INPUT, "invalid expert id: " + s);
    *layer = (int32_t)atoi(strip(ls).c_str());
    *expert = (int32_t)atoi(strip(es).c_str());
    return EK_OK;
}

ek_status ek_expert_id_format(const char *model, int32_t layer, int32_t expert, char *out, size_t cap)
{
    if (!model || !out || layer < 0 || expert < 0) return wire_fail(EK_INVALID_INPUT, "bad argument");
    const int n = snprintf(out, cap, "%s/l%d-e%d", model, layer, expert);   // as_object_key (:88-90)
    if (n < 0 || (size_t)n >= cap) return wire_fail(EK_INVALID_INPUT, "id buffer too small");
    return EK_OK;
}

}  // extern "C"

// Walks the header once.  match(name) picks the wanted entry; the first hit in header order wins.
template <typename Match>
static ek_status st_lookup(const void *blob, size_t len, Match match, const char *what, ek_tensor_view *out)
{
    if (!blob || !out) return wire_fail(EK_INVALID_INPUT, "NULL argument");
    if (len < 8) return wire_fail(EK_INVALID_INPUT, "safetensors: blob shorter than its length prefix");
    uint64_t hlen = 0;
    memcpy(&hlen, blob, 8);   // little endian
    if (hlen > len - 8 || hlen > (100u << 20)) return wire_fail(EK_INVALID_INPUT, "safetensors: bad header length");
    const char *h = (const char *)blob + 8;
    const size_t data_len = len - 8 - (size_t)hlen;
    ekw::Cursor c{h, h + hlen};
    if (!c.eat('{')) return wire_fail(EK_INVALID_INPUT, "safetensors: header is not a JSON object");
    bool found = false;
    ekw::Entry hit;
    if (!c.eat('}')) {
        while (true) {
            std::string key;
            if (!c.string(key) || !c.eat(':')) return wire_fail(EK_INVALID_INPUT, "safetensors: malformed header");
            if (key == "__metadata__") {
                if (!c.skip()) return wire_fail(EK_INVALID_INPUT, "safetensors: malformed metadata");
            } else {
                ekw::Entry e;
                if (!ekw::parse_entry(c, e)) return wire_fail(EK_INVALID_INPUT, "safetensors: malformed tensor entry");
                if (!found && match(key)) { hit = e; found = true; }
            }
            if (c.eat(',')) continue;
            if (!c.eat('}')) return wire_fail(EK_INVALID_INPUT, "safetensors: malformed header");
            break;
        }
    }
    if (!found) return wire_fail(EK_WEIGHT_NOT_FOUND, std::string("safetensors: no tensor ") + what);
    const ekw::DtypeName *dn = nullptr;
    for (const auto &d : ekw::kDtypes) if (hit.dtype == d.name) dn = &d;
    if (!dn) return wire_fail(EK_INVALID_INPUT, "safetensors: unsupported dtype " + hit.dtype);
    if (hit.shape.size() > 4) return wire_fail(EK_INVALID_INPUT, "safetensors: rank above 4");
    int64_t elems = 1;
    for (int64_t d : hit.shape) {
        if (d != 0 && elems > INT64_MAX / d) return wire_fail(EK_INVALID_INPUT, "safetensors: shape overflow");
        elems *= d;
    }
    if (hit.begin < 0 || hit.end < hit.begin || (uint64_t)hit.end > data_len ||
        elems > INT64_MAX / dn->size || hit.end - hit.begin != elems * dn->size)
        return wire_fail(EK_INVALID_INPUT, "safetensors: data_offsets do not match dtype and shape");
    out->data = h + hlen + hit.begin;
    out->rank = (int32_t)hit.shape.size();
    for (int i = 0; i < 4; ++i) out->shape[i] = i < out->rank ? hit.shape[i] : 1;
    out->dtype = dn->dtype;
    out->nbytes = hit.end - hit.begin;
    return EK_OK;
}

extern "C" {

static bool ends_with(const std::string &s, const char *suffix)
{
    const size_t n = strlen(suffix);
    return s.size() >= n && memcmp(s.data() + s.size() - n, suffix, n) == 0;
}

ek_status ek_safetensors_find(const void *blob, size_t len, const char *name, ek_tensor_view *out)
{
    if (!name) return wire_fail(EK_INVALID_INPUT, "NULL argument");
    return st_lookup(blob, len, [&](const std::string &k) { return k == name; }, name, out);
}

ek_status ek_safetensors_find_suffix(const void *blob, size_t len, const char *const *suffixes,
                                     int32_t n_suffixes, ek_tensor_view *out)
{
    if (!suffixes || n_suffixes < 1) return wire_fail(EK_INVALID_INPUT, "NULL argument");
    for (int i = 0; i < n_suffixes; ++i) if (!suffixes[i]) return wire_fail(EK_INVALID_INPUT, "NULL suffix");
    return st_lookup(blob, len,
                     [&](const std::string &k) {
                         for (int i = 0; i < n_suffixes; ++i) if (ends_with(k, suffixes[i])) return true;
                         return false;
                     },
                     suffixes[0], out);
}

// One matrix of an expert blob: the weight by suffix (ExpertWeight::from_safetensor,
// ffn/meta.rs:57-63) and, if the blob carries one, its scale "<weight name>_scale_inv"
// (ek-db/src/safetensor/transformer.rs:258-270) or "<weight name>_scale".
static ek_status blob_matrix(const void *blob, size_t len, const char *s1, const char *s2, const char *what,
                             ek_weight_desc *d)
{
    const char *sfx[2] = {s1, s2};
    ek_tensor_view w;
    ek_status st = ek_safetensors_find_suffix(blob, len, sfx, 2, &w);
    if (st == EK_WEIGHT_NOT_FOUND) return wire_fail(EK_WEIGHT_NOT_FOUND, what);
    if (st != EK_OK) return st;
    if (w.rank != 2) return wire_fail(EK_INVALID_INPUT, std::string(what) + ": weight is not a matrix");
    d->ptr = w.data; d->rows = w.shape[0]; d->cols = w.shape[1]; d->dtype = w.dtype; d->mem = EK_HOST;
    d->scale = nullptr; d->scale_dtype = EK_F32; d->scale_kind = EK_SCALE_NONE;
    const std::string a1 = std::string(s1) + "_scale_inv", a2 = std::string(s2) + "_scale_inv";
    const std::string b1 = std::string(s1) + "_scale", b2 = std::string(s2) + "_scale";
    const char *ssfx[4] = {a1.c_str(), a2.c_str(), b1.c_str(), b2.c_str()};
    ek_tensor_view sc;
    st = ek_safetensors_find_suffix(blob, len, ssfx, 4, &sc);
    if (st == EK_WEIGHT_NOT_FOUND) return EK_OK;
    if (st != EK_OK) return st;
    d->scale = sc.data;
    d->scale_dtype = sc.dtype;
    if (sc.rank == 1 && sc.shape[0] == d->rows) d->scale_kind = EK_SCALE_PER_CHANNEL;
    else if (sc.rank == 2 && sc.shape[0] == (d->rows + 127) / 128 && sc.shape[1] == (d->cols + 127) / 128)
        d->scale_kind = EK_SCALE_BLOCK128;
    else return wire_fail(EK_INVALID_INPUT, std::string(what) + ": scale tensor has neither [rows] nor [rows/128, cols/128] shape");
    return EK_OK;
}

ek_status ek_layer_set_expert_safetensors(ek_layer *layer, int32_t expert, const void *blob, size_t len)
{
    try {
        ek_weight_desc up, gate, down;
        ek_status st = blob_matrix(blob, len, "w1.weight", "up_proj.weight", "w1/up_w", &up);
        if (st != EK_OK) return st;
        st = blob_matrix(blob, len, "w2.weight", "down_proj.weight", "w2/down_w", &down);
        if (st != EK_OK) return st;
        st = blob_matrix(blob, len, "w3.weight", "gate_proj.weight", "w3/gate_w", &gate);
        if (st != EK_OK) return st;
        return ek_layer_set_expert(layer, expert, &up, &gate, &down);
    } catch (const std::exception &ex) {
        return wire_fail(EK_INTERNAL, std::string("exception: ") + ex.what());
    } catch (...) {
        return wire_fail(EK_INTERNAL, "unknown exception");
    }
}

static std::string st_header(const char *name, int32_t dtype, int32_t rank, const int64_t *shape, int64_t nbytes)
{
    const char *dn = nullptr;
    for (const auto &d : ekw::kDtypes) if (d.dtype == dtype) dn = d.name;
    std::string h = std::string("{\"") + name + "\":{\"dtype\":\"" + (dn ? dn : "?") + "\",\"shape\":[";
    for (int i = 0; i < rank; ++i) h += (i ? "," : "") + std::to_string(shape[i]);
    h += "],\"data_offsets\":[0," + std::to_string(nbytes) + "]}}";
    while (h.size() % 8) h.push_back(' ');   // the format pads the header to 8 bytes with spaces
    return h;
}

static int64_t st_nbytes(int32_t dtype, int32_t rank, const int64_t *shape)
{
    int64_t es = 0;
    for (const auto &d : ekw::kDtypes) if (d.dtype == dtype) es = d.size;
    if (!es || rank < 0 || rank > 4 || (rank && !shape)) return -1;
    int64_t n = es;
    for (int i = 0; i < rank; ++i) { if (shape[i] < 0) return -1; n *= shape[i]; }
    return n;
}

size_t ek_safetensors_size(const char *name, int32_t dtype, int32_t rank, const int64_t *shape)
{
    const int64_t nb = st_nbytes(dtype, rank, shape);
    if (nb < 0 || !name) return 0;
    return 8 + st_header(name, dtype, rank, shape, nb).size() + (size_t)nb;
}

ek_status ek_safetensors_emit(const char *name, int32_t dtype, int32_t rank, const int64_t *shape,
                              const void *data, void *out, size_t cap, size_t *written)
{
    const int64_t nb = st_nbytes(dtype, rank, shape);
    if (nb < 0 || !name || !out || (nb && !data)) return wire_fail(EK_INVALID_INPUT, "safetensors: bad tensor description");
    const std::string h = st_header(name, dtype, rank, shape, nb);
    const size_t total = 8 + h.size() + (size_t)nb;
    if (cap < total) return wire_fail(EK_INVALID_INPUT, "safetensors: output buffer too small");
    const uint64_t hlen = h.size();
    memcpy(out, &hlen, 8);
    memcpy((char *)out + 8, h.data(), h.size());
    if (nb) memcpy((char *)out + 8 + h.size(), data, (size_t)nb);
    if (written) *written = total;
    return EK_OK;
}

// One request: checks and views.  *rows == 0 is legal.
static ek_status open_request(ek_layer *layer, const char *expert_id, const void *req, size_t req_len,
                              int32_t *expert, ek_tensor_view *tv)
{
    int64_t hid = 0;
    int32_t act = 0, nexp = 0;
    ek_status st = ek_layer_describe(layer, &hid, nullptr, &nexp, nullptr, &act);
    if (st != EK_OK) return st;
    int32_t lyr = 0;
    st = ek_expert_id_parse(expert_id, &lyr, expert);
    if (st != EK_OK) return st;
    if (*expert >= nexp) return wire_fail(EK_EXPERT_NOT_FOUND, std::string("expert not found: ") + expert_id);
    st = ek_safetensors_find(req, req_len, "data", tv);
    if (st != EK_OK) return st;
    if (tv->rank != 2) return wire_fail(EK_INVALID_INPUT, "request tensor must have rank 2 (ffn/mod.rs:45)");
    if (tv->shape[1] != hid) return wire_fail(EK_INVALID_INPUT, "request tensor's last dimension is not the hidden size");
    if (tv->dtype != act) return wire_fail(EK_INVALID_INPUT, "request tensor's dtype is not the layer's activation dtype");
    return EK_OK;
}

ek_status ek_worker_forward(ek_layer *layer, const char *expert_id, const void *req, size_t req_len,
                            void *resp, size_t resp_cap, size_t *resp_len)
{
    const char *ids[1] = {expert_id};
    const void *reqs[1] = {req};
    void *resps[1] = {resp};
    return ek_worker_forward_batch(layer, 1, ids, reqs, &req_len, resps, &resp_cap, resp_len);
}

ek_status ek_worker_forward_batch(ek_layer *layer, int32_t n_calls, const char *const *expert_ids,
                                  const void *const *reqs, const size_t *req_lens, void *const *resps,
                                  const size_t *resp_caps, size_t *resp_lens)
{
    try {
        if (!layer || n_calls < 0 || (n_calls && (!expert_ids || !reqs || !req_lens || !resps || !resp_caps || !resp_lens)))
            return wire_fail(EK_INVALID_INPUT, "NULL argument");
        std::vector<int32_t> experts(n_calls);
        std::vector<int64_t> rows(n_calls);
        std::vector<const void *> xs(n_calls);
        std::vector<void *> outs(n_calls);
        std::vector<size_t> hdr(n_calls);
        int32_t act = 0;
        ek_status st = ek_layer_describe(layer, nullptr, nullptr, nullptr, nullptr, &act);
        if (st != EK_OK) return st;
        for (int i = 0; i < n_calls; ++i) {
            ek_tensor_view tv;
            st = open_request(layer, expert_ids[i], reqs[i], req_lens[i], &experts[i], &tv);
            if (st != EK_OK) return st;
            rows[i] = tv.shape[0];
            xs[i] = tv.data;
            // the response header is known before the data: write it now, compute straight into place
            const int64_t shape[2] = {tv.shape[0], tv.shape[1]};
            const std::string h = st_header("data", act, 2, shape, tv.nbytes);
            const size_t total = 8 + h.size() + (size_t)tv.nbytes;
            if (!resps[i] || resp_caps[i] < total) return wire_fail(EK_INVALID_INPUT, "response buffer too small");
            const uint64_t hlen = h.size();
            memcpy(resps[i], &hlen, 8);
            memcpy((char *)resps[i] + 8, h.data(), h.size());
            hdr[i] = 8 + h.size();
            outs[i] = (char *)resps[i] + hdr[i];
            resp_lens[i] = total;
        }
        st = ek_layer_experts_forward(layer, n_calls, experts.data(), xs.data(), rows.data(), outs.data(), EK_HOST, nullptr);
        return st;
    } catch (const std::exception &ex) {
        return wire_fail(EK_INTERNAL, std::string("exception: ") + ex.what());
    } catch (...) {
        return wire_fail(EK_INTERNAL, "unknown exception");
    }
}

}  // extern "C"
