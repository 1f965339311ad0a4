// cybq.hpp - C++ host layer over the C ABI in cybq.h (header only).
//
// The reference's host side is compiled code: a runtime crate that maps a
// .model file, walks a graph IR and calls a compute backend once per node
// (/root/reference/decide/pipeline.md:28-30,51;
// /root/reference/decide/model-lifecycle.md:25-26,37).  That crate is outside
// the reference tree, so this header mirrors the seam with the facts the tree
// does give: a backend object created once
// (/root/reference/shell/src/worlds/soma_bridge.rs:65), tensors handed over at
// model load and kept by HF-style name
// (/root/reference/shell/src/worlds/models/mod.rs:7-8,386), one call per
// quantised-matmul node, errors as values
// (/root/reference/shell/src/worlds/soma_bridge.rs:322-333).
//
// Nothing here computes anything: every method forwards to libcybq.
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "cybq.h"

namespace cybq {

// Result of every fallible call: status 0 = ok, otherwise a cybq_status and text.
struct Status {
    int code = CYBQ_OK;
    std::string text;
    bool ok() const { return code == CYBQ_OK; }
    explicit operator bool() const { return ok(); }
};

// Graph-IR node of the op: y = x * dequant(w)^T.  `w` names the tensor,
// `x` / `y` name edges.  (Stand-in: the reference's node fields are not visible.)
struct QMatMulNode {
    std::string w, x, y;
    cybq_quant quant = CYBQ_Q4;
    int group = CYBQ_GROUP;
    int64_t M = 1, N = 0, K = 0;
    cybq_epilogue epilogue = CYBQ_EPI_NONE;   // fused op behind the linear
    std::string residual;                      // edge added to the output (CYBQ_EPI_ADD)
    std::string norm_gamma;                    // edge holding gamma [K]: RMSNorm folded into the x load ("" = none)
    float norm_eps = 1e-5f;
};

// A device buffer bound to an edge name: pointer, element type, rows.
struct Edge {
    void* ptr = nullptr;
    cybq_dtype dtype = CYBQ_F16;
    int64_t rows = 0, cols = 0;
};

class Backend;

class Weight {
public:
    Weight() = default;
    Weight(const Weight&) = delete;
    Weight& operator=(const Weight&) = delete;
    Weight(Weight&& o) noexcept { *this = std::move(o); }
    Weight& operator=(Weight&& o) noexcept
    {
        if (this != &o) { reset(); ctx_ = o.ctx_; h_ = o.h_; o.h_ = nullptr; }
        return *this;
    }
    ~Weight() { reset(); }
    const cybq_weight* get() const { return h_; }
    explicit operator bool() const { return h_ != nullptr; }
    int64_t rows() const { int64_t n = 0; if (h_) cybq_weight_info(h_, nullptr, &n, nullptr, nullptr); return n; }
    int64_t cols() const { int64_t k = 0; if (h_) cybq_weight_info(h_, nullptr, nullptr, &k, nullptr); return k; }
    int quant() const { int q = 0; if (h_) cybq_weight_info(h_, &q, nullptr, nullptr, nullptr); return q; }

private:
    friend class Backend;
    void reset() { if (h_) { cybq_weight_free(ctx_, h_); h_ = nullptr; } }
    cybq_ctx* ctx_ = nullptr;
    cybq_weight* h_ = nullptr;
};

class Backend {
public:
    // never throws: check ok() / status()
    explicit Backend(int device = 0) { st_ = wrap(cybq_init(device, &ctx_)); }
    Backend(const Backend&) = delete;
    Backend& operator=(const Backend&) = delete;
    ~Backend()
    {
        weights_.clear();            // handles are freed while the context is alive
        if (ctx_) cybq_destroy(ctx_);
    }
    bool ok() const { return ctx_ != nullptr; }
    const Status& status() const { return st_; }

    // model load: one call per quantised tensor; `q` / `scales` point into the mapped file
    Status load(const std::string& name, cybq_quant quant, cybq_layout layout, int64_t N, int64_t K,
                const void* q, const void* scales)
    {
        Weight w;
        w.ctx_ = ctx_;
        Status s = wrap(cybq_weight_upload(ctx_, quant, layout, N, K, q, scales, &w.h_));
        if (s) weights_[name] = std::move(w);
        return s;
    }
    // gate and up projections of one FFN as a single weight for CYBQ_EPI_SWIGLU
    Status fuse_pairs(const std::string& name, const std::string& gate, const std::string& up)
    {
        const Weight *g = find(gate), *u = find(up);
        if (!g || !u) return fail(CYBQ_ERR_INVALID, "gate / up not loaded");
        Weight w;
        w.ctx_ = ctx_;
        Status s = wrap(cybq_weight_fuse_pairs(ctx_, g->get(), u->get(), &w.h_));
        if (s) weights_[name] = std::move(w);
        return s;
    }
    void unload(const std::string& name) { weights_.erase(name); }
    const Weight* find(const std::string& name) const
    {
        auto it = weights_.find(name);
        return it == weights_.end() ? nullptr : &it->second;
    }

    Status set_prefill_mode(cybq_prefill_mode m) { return wrap(cybq_set_prefill_mode(ctx_, m)); }

    Status matmul(const Weight& w, const void* x, cybq_dtype xdt, int64_t M, void* y, cybq_dtype ydt,
                  void* stream = nullptr)
    {
        return wrap(cybq_matmul(ctx_, w.get(), x, xdt, M, y, ydt, stream));
    }
    Status matmul_ex(const Weight& w, const void* x, cybq_dtype xdt, int64_t M, void* y, cybq_dtype ydt,
                     cybq_epilogue epilogue, const void* residual, void* stream = nullptr)
    {
        return wrap(cybq_matmul_ex(ctx_, w.get(), x, xdt, M, y, ydt, epilogue, residual, stream));
    }
    Status matmul_norm(const Weight& w, const void* x, cybq_dtype xdt, int64_t M, const void* gamma, cybq_dtype gdt,
                       float eps, void* y, cybq_dtype ydt, cybq_epilogue epilogue = CYBQ_EPI_NONE,
                       const void* residual = nullptr, void* stream = nullptr)
    {
        return wrap(cybq_matmul_norm(ctx_, w.get(), x, xdt, M, gamma, gdt, eps, y, ydt, epilogue, residual, stream));
    }
    Status dequant(const Weight& w, float* out, void* stream = nullptr)
    {
        return wrap(cybq_dequant(ctx_, w.get(), out, stream));
    }

    // one graph node; shape fields of the node are checked against the loaded tensor
    Status run(const QMatMulNode& node, const std::map<std::string, Edge>& edges, void* stream = nullptr)
    {
        if (node.group != CYBQ_GROUP) return fail(CYBQ_ERR_SHAPE, "group must be 32");
        const Weight* w = find(node.w);
        if (!w) return fail(CYBQ_ERR_INVALID, "weight '" + node.w + "' not loaded");
        if ((node.N && node.N != w->rows()) || (node.K && node.K != w->cols()) || (int)node.quant != w->quant())
            return fail(CYBQ_ERR_SHAPE, "node '" + node.w + "' does not match the loaded tensor");
        auto xi = edges.find(node.x), yi = edges.find(node.y);
        if (xi == edges.end() || yi == edges.end()) return fail(CYBQ_ERR_INVALID, "edge not bound");
        if (xi->second.rows < node.M || yi->second.rows < node.M) return fail(CYBQ_ERR_SHAPE, "edge has too few rows");
        if (Status s = check_cols(*w, node, xi->second, yi->second); !s) return s;
        const void* res = nullptr;
        if (node.epilogue == CYBQ_EPI_ADD) {
            auto ri = edges.find(node.residual);
            if (ri == edges.end() || ri->second.dtype != yi->second.dtype || ri->second.rows < node.M ||
                ri->second.cols != yi->second.cols)
                return fail(CYBQ_ERR_INVALID, "residual edge not bound, of another type or of another shape");
            res = ri->second.ptr;
        }
        if (!node.norm_gamma.empty()) {
            auto gi = edges.find(node.norm_gamma);
            if (gi == edges.end()) return fail(CYBQ_ERR_INVALID, "gamma edge not bound");
            if (gi->second.rows * gi->second.cols != w->cols()) return fail(CYBQ_ERR_SHAPE, "gamma must hold K elements");
            return matmul_norm(*w, xi->second.ptr, xi->second.dtype, node.M, gi->second.ptr, gi->second.dtype, node.norm_eps,
                               yi->second.ptr, yi->second.dtype, node.epilogue, res, stream);
        }
        return matmul_ex(*w, xi->second.ptr, xi->second.dtype, node.M, yi->second.ptr, yi->second.dtype, node.epilogue,
                         res, stream);
    }

    // a whole step: the nodes are resolved once, then launched back to back from native code
    Status run_all(const std::vector<QMatMulNode>& nodes, const std::map<std::string, Edge>& edges,
                   void* stream = nullptr)
    {
        if (nodes.empty()) return Status{};
        std::vector<const cybq_weight*> ws;
        std::vector<const void*> xs, rs, gs;
        std::vector<void*> ys;
        std::vector<int> es;
        bool normed = false;                  // one gamma type and one eps for the whole list
        cybq_dtype gdt = CYBQ_F32;
        float eps = 0.f;
        auto x0i = edges.find(nodes[0].x), y0i = edges.find(nodes[0].y);
        if (x0i == edges.end() || y0i == edges.end()) return fail(CYBQ_ERR_INVALID, "unresolved node '" + nodes[0].w + "'");
        const Edge &x0 = x0i->second, &y0 = y0i->second;
        for (const auto& n : nodes) {
            const Weight* w = find(n.w);
            auto xi = edges.find(n.x), yi = edges.find(n.y);
            if (!w || xi == edges.end() || yi == edges.end()) return fail(CYBQ_ERR_INVALID, "unresolved node '" + n.w + "'");
            if (xi->second.dtype != x0.dtype || yi->second.dtype != y0.dtype || n.M != nodes[0].M)
                return fail(CYBQ_ERR_INVALID, "run_all needs one M and one dtype pair");
            if (xi->second.rows < n.M || yi->second.rows < n.M) return fail(CYBQ_ERR_SHAPE, "edge has too few rows");
            if (Status s = check_cols(*w, n, xi->second, yi->second); !s) return s;
            const void* gam = nullptr;
            if (!n.norm_gamma.empty()) {
                auto gi = edges.find(n.norm_gamma);
                if (gi == edges.end()) return fail(CYBQ_ERR_INVALID, "gamma edge of '" + n.w + "' not bound");
                if (gi->second.rows * gi->second.cols != w->cols()) return fail(CYBQ_ERR_SHAPE, "gamma must hold K elements");
                if (normed && (gi->second.dtype != gdt || n.norm_eps != eps))
                    return fail(CYBQ_ERR_INVALID, "run_all needs one gamma type and one eps: use run()");
                normed = true;
                gdt = gi->second.dtype;
                eps = n.norm_eps;
                gam = gi->second.ptr;
            }
            gs.push_back(gam);
            const void* res = nullptr;
            if (n.epilogue == CYBQ_EPI_ADD) {
                auto ri = edges.find(n.residual);
                if (ri == edges.end() || ri->second.dtype != y0.dtype) return fail(CYBQ_ERR_INVALID, "residual of '" + n.w + "' not bound");
                res = ri->second.ptr;
            }
            ws.push_back(w->get());
            xs.push_back(xi->second.ptr);
            ys.push_back(yi->second.ptr);
            es.push_back((int)n.epilogue);
            rs.push_back(res);
        }
        if (normed)
            return wrap(cybq_matmul_many_norm(ctx_, (int64_t)nodes.size(), ws.data(), xs.data(), gs.data(), gdt, eps, ys.data(),
                                              es.data(), rs.data(), x0.dtype, nodes[0].M, y0.dtype, stream));
        return wrap(cybq_matmul_many_ex(ctx_, (int64_t)nodes.size(), ws.data(), xs.data(), ys.data(), es.data(), rs.data(),
                                        x0.dtype, nodes[0].M, y0.dtype, stream));
    }

private:
    // an edge's columns must be what the weight reads (K) and writes (N, or N / 2 behind SwiGLU)
    Status check_cols(const Weight& w, const QMatMulNode& node, const Edge& x, const Edge& y)
    {
        if (!x.ptr || !y.ptr) return fail(CYBQ_ERR_INVALID, "edge without a buffer");
        const int64_t n_out = node.epilogue == CYBQ_EPI_SWIGLU ? w.rows() / 2 : w.rows();
        if (x.cols != w.cols() || y.cols != n_out)
            return fail(CYBQ_ERR_SHAPE, "edges of node '" + node.w + "' do not have the weight's K / N columns");
        return Status{};
    }
    Status wrap(int rc)
    {
        Status s;
        s.code = rc;
        if (rc != CYBQ_OK) {
            s.text = cybq_strerror(rc);
            const char* d = ctx_ ? cybq_last_error(ctx_) : "";
            if (d && *d) s.text += std::string(": ") + d;
        }
        return s;
    }
    Status fail(int rc, const std::string& why)
    {
        Status s;
        s.code = rc;
        s.text = std::string(cybq_strerror(rc)) + ": " + why;
        return s;
    }
    cybq_ctx* ctx_ = nullptr;
    Status st_;
    std::map<std::string, Weight> weights_;
};

}  // namespace cybq
