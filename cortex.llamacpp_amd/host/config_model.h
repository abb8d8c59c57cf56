// config_model.h — what the loaders of the folder models (config.json + model.safetensors, bf16 weights) share: reading the configuration, checking every
// tensor against it on the way to the device, and laying out the order of layer runs with its looped span.  One loader per design (novorax.cc, fidepel.cc,
// tuterax.cc, dinilorn.cc);
// config_model_load picks it by the configuration's "architecture".
#pragma once

#include <algorithm>
#include <cstring>
#include <string>
#include <vector>

#include "json.h"
#include "runtime.h"
#include "safetensors.h"

namespace mi355 {

struct Bf16Loader {
    SafeTensorsFile st;
    Model *m = nullptr;
    std::string err;
    uint64_t bytes = 0;

    void *dev(const void *host, size_t n) {
        if (!err.empty()) return nullptr;
        void *p = nullptr;
        if (hipMalloc(&p, n ? n : 16) != hipSuccess) { err = "device allocation of " + std::to_string(n) + " bytes failed"; return nullptr; }
        m->arenas.push_back((uint8_t *)p);
        if (n && hipMemcpy(p, host, n, hipMemcpyHostToDevice) != hipSuccess) { err = "upload failed"; return nullptr; }
        bytes += n;
        return p;
    }
    const SafeTensor *need(const std::string &name, const char *dtype, std::initializer_list<int64_t> shape) {
        if (!err.empty()) return nullptr;
        const SafeTensor *t = st.find(name);
        if (!t) { err = "tensor '" + name + "' missing"; return nullptr; }
        if (t->dtype != dtype) { err = "tensor '" + name + "' is " + t->dtype + ", expected " + dtype; return nullptr; }
        if (t->shape.size() != shape.size() || !std::equal(shape.begin(), shape.end(), t->shape.begin())) {
            std::string want, have;
            for (int64_t d : shape) want += (want.empty() ? "" : ", ") + std::to_string(d);
            for (int64_t d : t->shape) have += (have.empty() ? "" : ", ") + std::to_string(d);
            err = "tensor '" + name + "' has shape [" + have + "], the configuration asks for [" + want + "]";
            return nullptr;
        }
        return t;
    }
    // several [rows_i][K] bf16 tensors under each other as one device matrix
    BfMat rows(const std::vector<std::pair<std::string, int>> &parts, int K) {
        BfMat o;
        std::vector<unsigned short> host;
        for (const auto &pr : parts) {
            const SafeTensor *t = need(pr.first, "BF16", {pr.second, K});
            if (!t) return o;
            const unsigned short *s = (const unsigned short *)t->data;
            host.insert(host.end(), s, s + (size_t)pr.second * K);
            o.N += pr.second;
        }
        o.K = K;
        o.w = (unsigned short *)dev(host.data(), host.size() * 2);
        return o;
    }
    static float widen(unsigned short b) { const uint32_t u = (uint32_t)b << 16; float f; memcpy(&f, &u, 4); return f; }
    float *vec(const std::string &name, int n) {
        const SafeTensor *t = need(name, "BF16", {n});
        if (!t) return nullptr;
        std::vector<float> h((size_t)n);
        const unsigned short *s = (const unsigned short *)t->data;
        for (int i = 0; i < n; i++) h[(size_t)i] = widen(s[i]);
        return (float *)dev(h.data(), h.size() * 4);
    }
    // rows of a [rows][K] tensor whose row count the configuration does not name (a low-rank projection's inner size): -1 (err set) if absent or not 2-d
    int rows_of(const std::string &name, int K) {
        if (!err.empty()) return -1;
        const SafeTensor *t = st.find(name);
        if (!t) { err = "tensor '" + name + "' missing"; return -1; }
        if (t->shape.size() != 2 || t->shape[1] != K || t->shape[0] < 1 || t->shape[0] > (1 << 24)) { err = "tensor '" + name + "' must be [rows][" + std::to_string(K) + "]"; return -1; }
        return (int)t->shape[0];
    }
    // several [rows_i][K] bf16 tensors under each other, widened to f32 (small per-channel tables a kernel reads as floats)
    float *rows_f32(const std::vector<std::pair<std::string, int>> &parts, int K) {
        std::vector<float> host;
        for (const auto &pr : parts) {
            const SafeTensor *t = need(pr.first, "BF16", {pr.second, K});
            if (!t) return nullptr;
            const unsigned short *s = (const unsigned short *)t->data;
            for (size_t i = 0; i < (size_t)pr.second * K; i++) host.push_back(widen(s[i]));
        }
        return (float *)dev(host.data(), host.size() * 4);
    }
    // a tensor that holds ONE number, as n copies of it: a norm weight shared by all coordinates takes the kernels' per-coordinate form
    float *scalar_as_vec(const std::string &name, int n) {
        const SafeTensor *t = need(name, "BF16", {});
        if (!t) return nullptr;
        std::vector<float> h((size_t)n, widen(*(const unsigned short *)t->data));
        return (float *)dev(h.data(), h.size() * 4);
    }
    // the embedding table with the row stride launch_get_rows expects
    BfMat embedding(const std::string &name, int V, int W) {
        BfMat o;
        const SafeTensor *t = need(name, "BF16", {V, W});
        if (!t) return o;
        const size_t rb = dev_row_bytes(T_BF16, W);
        std::vector<uint8_t> host((size_t)V * rb, 0);
        for (int r = 0; r < V; r++) memcpy(host.data() + (size_t)r * rb, t->data + (size_t)r * W * 2, (size_t)W * 2);
        o.w = (unsigned short *)dev(host.data(), host.size());
        o.N = V; o.K = W;
        return o;
    }
};

inline bool cfg_positive(std::string &err, const char *what, int64_t v, int64_t hi = 1 << 24) {
    if (v >= 1 && v <= hi) return true;
    err = std::string("configuration: ") + what + " = " + std::to_string(v) + " is out of range";
    return false;
}

// The order of layer runs from the configuration's "loop" {start, stop, times}: layers before the span once, the span `times` times with the same weights,
// the rest once.  on_run(layer, pass): pass >= 0 for the first layer of pass `pass` of the span, -1 elsewhere.  false (err set) for a span out of range.
template <class F>
bool cfg_layer_runs(const Json &loop, int n_layer, std::string &err, int &times_out, F on_run) {
    int a = 0, b = 0, times = 0;
    if (loop.is_object()) {
        a = (int)loop["start"].as_int(0); b = (int)loop["stop"].as_int(0); times = (int)loop["times"].as_int(1);
        if (a < 0 || b > n_layer || times < 0 || times > 4096) { err = "configuration: loop start / stop / times out of range"; return false; }
        if (b <= a || times < 1) { a = b = 0; times = 0; }
    }
    for (int i = 0; i < a; i++) on_run(i, -1);
    for (int t = 0; t < times; t++) for (int i = a; i < b; i++) on_run(i, i == a ? t : -1);
    for (int i = b; i < n_layer; i++) on_run(i, -1);
    times_out = times;
    return true;
}

// from this many (token, rank) pairs on a routed feed-forward groups the pairs by expert and runs every expert's rows as one batch (fidepel.cc)
bool nvx_routed_as_groups(const NvxLayer &L, int T);

// the designs' loaders: cfg is the parsed config.json of `dir`, ld has model.safetensors open and ld.m set
Model *novorax_build(const Json &cfg, const std::string &dir, Bf16Loader &ld, std::string &err, int &status);
Model *fidepel_build(const Json &cfg, const std::string &dir, Bf16Loader &ld, std::string &err, int &status);
Model *tuterax_build(const Json &cfg, const std::string &dir, Bf16Loader &ld, std::string &err, int &status);
Model *dinilorn_build(const Json &cfg, const std::string &dir, Bf16Loader &ld, std::string &err, int &status);

}  // namespace mi355
