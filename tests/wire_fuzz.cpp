// Mutated safetensors blobs and expert ids through the wire parser; built with the host compiler's address and
// undefined-behaviour sanitizers by tests/test_wire_cpu.py (no GPU call is made).  Every blob is handed over as an
// exact-size heap copy, so a read past its end is reported; views must lie inside the blob.
#include "ek_hip.h"
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>
static std::vector<uint8_t> blob_of(const std::string &header, size_t payload)
{
    std::vector<uint8_t> b(8 + header.size() + payload);
    uint64_t n = header.size();
    memcpy(b.data(), &n, 8);
    memcpy(b.data() + 8, header.data(), header.size());
    for (size_t i = 0; i < payload; ++i) b[8 + header.size() + i] = (uint8_t)i;
    return b;
}
int main(int argc, char **argv)
{
    const long iters = argc > 1 ? atol(argv[1]) : 200000;
    std::mt19937_64 rng(12345);
    std::vector<std::vector<uint8_t>> good;
    good.push_back(blob_of("{\"data\":{\"dtype\":\"BF16\",\"shape\":[5,64],\"data_offsets\":[0,640]}}", 640));
    good.push_back(blob_of("{\"__metadata__\":{\"k\":\"v\"},\"a.w1.weight\":{\"dtype\":\"F32\",\"shape\":[8,8],\"data_offsets\":[0,256]},\"data\":{\"dtype\":\"I8\",\"shape\":[3,16],\"data_offsets\":[256,304]}}   ", 304));
    good.push_back(blob_of("{\"m.layers.3.mlp.experts.7.up_proj.weight\":{\"dtype\":\"F8_E4M3\",\"shape\":[4,4],\"data_offsets\":[0,16]},\"m.layers.3.mlp.experts.7.up_proj.weight_scale_inv\":{\"dtype\":\"F32\",\"shape\":[1,1],\"data_offsets\":[16,20]}}", 20));
    // no payload: the header's end is the blob's end, so a read past the header is a read past the allocation
    good.push_back(blob_of("{\"data\":{\"dtype\":\"BF16\",\"shape\":[0,8],\"data_offsets\":[0,0]}}", 0));
    good.push_back(blob_of("{\"x\":{\"dtype\":\"F16\",\"shape\":[0],\"data_offsets\":[0,0]},\"__metadata__\":{\"a\":\"b\"}} ", 0));
    const char *suffixes[] = {"w1.weight", "up_proj.weight", "up_proj.weight_scale_inv", "data"};
    long ok = 0, bad = 0;
    for (long it = 0; it < iters; ++it) {
        std::vector<uint8_t> b = good[it % good.size()];
        uint64_t hl; memcpy(&hl, b.data(), 8);
        switch (rng() % 8) {
        case 0: b.resize(rng() % (b.size() + 1)); break;
        case 1: for (int k = 1 + rng() % 5; k--;) b[8 + rng() % hl] = (uint8_t)rng(); break;
        case 2: { uint64_t v = rng() >> (rng() % 64); memcpy(b.data(), &v, 8); break; }
        case 3: { size_t pos = 8 + rng() % hl; b.insert(b.begin() + pos, 1 + rng() % 30, (uint8_t)'9'); break; }
        case 4: for (auto &c : b) c = (uint8_t)rng(); break;
        case 5: { size_t a = 8 + rng() % hl, n = 1 + rng() % 12; if (a + n > b.size()) n = b.size() - a; b.erase(b.begin() + a, b.begin() + a + n); break; }
        case 6: { const char toks[] = "{}[]\",:-\\u"; for (int k = 1 + rng() % 8; k--;) b[8 + rng() % hl] = (uint8_t)toks[rng() % (sizeof toks - 1)]; break; }
        default: { uint64_t v = hl + (int64_t)(rng() % 17) - 8; memcpy(b.data(), &v, 8); break; }
        }
        // an exact-size heap copy so that any read past the end is seen
        uint8_t *p = (uint8_t *)malloc(b.size() ? b.size() : 1);
        memcpy(p, b.data(), b.size());
        ek_tensor_view v;
        ek_status st = ek_safetensors_find(p, b.size(), "data", &v);
        if (st == EK_OK) {
            ++ok;
            if ((const uint8_t *)v.data < p || (const uint8_t *)v.data + v.nbytes > p + b.size()) { printf("view outside blob it=%ld\n", it); return 1; }
            volatile uint8_t sink = 0;
            for (int64_t i = 0; i < v.nbytes; ++i) sink ^= ((const uint8_t *)v.data)[i];
        } else ++bad;
        st = ek_safetensors_find_suffix(p, b.size(), suffixes, 4, &v);
        if (st == EK_OK && ((const uint8_t *)v.data < p || (const uint8_t *)v.data + v.nbytes > p + b.size())) { printf("suffix view outside blob it=%ld\n", it); return 1; }
        free(p);
        // expert ids
        std::string id = "model-x/l12-e345";
        for (int k = rng() % 4; k--;) id[rng() % id.size()] = (char)(rng() % 128);
        if (rng() % 5 == 0) id.resize(rng() % (id.size() + 1));
        if (rng() % 7 == 0) id += std::string(rng() % 40, '9');
        char *idp = strdup(id.c_str());
        int32_t l, e;
        ek_expert_id_parse(idp, &l, &e);
        free(idp);
        char out[24];
        ek_expert_id_format("some-model", (int32_t)rng(), (int32_t)rng(), out, rng() % sizeof out);
    }
    printf("ok=%ld bad=%ld\n", ok, bad);
    return 0;
}
