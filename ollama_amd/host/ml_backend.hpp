// C++ host-side mirror of the reference's tensor-backend interface for the Mulmat path, over the
// C ABI in include/mi_qmm.h.  The reference declares it in Go:
//   ml.Backend  /root/reference/ml/backend.go:16-33    Load / Get(name) / NewContext / Close
//   ml.Context  /root/reference/ml/backend.go:94-128   FromFloats / Compute / Close
//   ml.Tensor   /root/reference/ml/backend.go:130-153  Dim / Shape / Floats / Mulmat / MulmatFullPrec / MulmatID
//               /root/reference/ml/backend.go:159, :180 RMSNorm(ctx, weight, eps) / SILU(ctx, up)
// Same names, same argument meaning (ggml shapes: dimension 0 contiguous, W = [K, M], x = [K, N],
// W.Mulmat(ctx, x) = [M, N]) and the same error behaviour: tensor ops have no error return, so a
// failure throws (the Go interface panics).  Mulmat is lazy; Compute runs the pending nodes, sharing
// one activation quantization between all nodes that read the same x.  An RMSNorm or SILU(up) node that only
// products read is never materialized: it runs inside those products' quantization; gate.SILU(up) on two
// products of one x that nothing else reads runs as one call and the two products are not materialized.
#pragma once

#include <cstdint>
#include <cstring>
#include <map>
#include <set>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../include/mi_qmm.h"

namespace ollama_amd {

struct Error : std::runtime_error {
    int code;
    Error(int c, const std::string &what) : std::runtime_error(what), code(c) {}
};

inline void check(int rc) {
    if (rc != MI_QMM_OK) throw Error(rc, mi_qmm_last_error());
}

class Context;

class Tensor : public std::enable_shared_from_this<Tensor> {
public:
    int Dim(int n) const { return n < (int)shape_.size() ? (int)shape_[n] : 1; }
    const std::vector<int64_t> &Shape() const { return shape_; }
    int GGMLType() const { return type_; }
    // values in ggml order (dimension 0 contiguous); throws until Compute has produced them
    const std::vector<float> &Floats() const {
        if (!ready_) throw Error(MI_QMM_ERR_INVALID, "tensor has no data yet: call Context::Compute first");
        return data_;
    }
    // self = quantized weight [K, M], t2 = f32 activations [K, N] -> lazy [M, N]
    std::shared_ptr<Tensor> Mulmat(Context &ctx, const std::shared_ptr<Tensor> &t2);
    std::shared_ptr<Tensor> MulmatFullPrec(Context &ctx, const std::shared_ptr<Tensor> &t2) { return Mulmat(ctx, t2); }
    // self = expert stack [K, M, E], t2 = f32 [K, B, T] (B = 1 or n_used), ids = int32 [n_used, T] -> lazy
    // [M, n_used, T]: slot i of token t goes through expert ids[i, t] with activation row i mod B
    std::shared_ptr<Tensor> MulmatID(Context &ctx, const std::shared_ptr<Tensor> &t2, const std::shared_ptr<Tensor> &ids);
    const std::vector<int32_t> &Ints() const { return ints_; }
    // self = x [K, ...] f32, weight = [K] f32 or null -> lazy (x / sqrt(mean(x^2) + eps)) * weight along dimension 0
    std::shared_ptr<Tensor> RMSNorm(Context &ctx, const std::shared_ptr<Tensor> &weight, float eps);
    // self = gate, up: f32 of one shape -> lazy silu(gate) * up (ggml's swiglu)
    std::shared_ptr<Tensor> SILU(Context &ctx, const std::shared_ptr<Tensor> &up = nullptr);

    ~Tensor() { mi_qmm_weight_free(weight_); }

private:
    friend class Backend;
    friend class Context;
    std::vector<int64_t> shape_;
    int type_ = MI_QMM_TYPE_F32;
    mi_qmm_weight *weight_ = nullptr;
    std::vector<float> data_;
    std::vector<int32_t> ints_;          // values of an int32 tensor (FromInts)
    bool ready_ = false;
    Tensor *op_w_ = nullptr;             // pending Mulmat: weight
    std::shared_ptr<Tensor> op_x_;       // pending Mulmat: activations
    std::shared_ptr<Tensor> op_ids_;     // pending MulmatID: expert ids
    std::shared_ptr<Tensor> self_keep_;  // keeps the weight alive while a node refers to it
    int prod_ = MI_QMM_PRODUCE_NONE;     // pending RMSNorm / SILU(up): the producer,
    std::shared_ptr<Tensor> prod_src_;   //   its input,
    std::shared_ptr<Tensor> prod_aux_;   //   the norm weight (may be null) or up,
    float prod_eps_ = 0.f;               //   and eps
    bool absorbed_ = false;              // a product computed inside the SILU node that reads it
};

class Backend {
public:
    explicit Backend(int device = 0) { check(mi_qmm_init(device, &ctx_)); }
    ~Backend() { Close(); }
    Backend(const Backend &) = delete;
    Backend &operator=(const Backend &) = delete;

    // One GGUF tensor: type id, shape [K, M], M rows of K elements in GGUF block layout (what fs/ggml
    // hands out, /root/reference/fs/ggml/gguf.go:281-308).  The bytes are copied to the device.
    void Load(const std::string &name, int ggml_type, int64_t k, int64_t m, const void *gguf_bytes) {
        if (ggml_type == MI_QMM_TYPE_F32 && m == 1) {  // a norm weight, the operand of RMSNorm: stays on the host
            auto t = std::make_shared<Tensor>();
            t->shape_ = {k};
            t->data_.resize((size_t)k);
            std::memcpy(t->data_.data(), gguf_bytes, (size_t)k * sizeof(float));
            t->ready_ = true;
            tensors_[name] = t;
            return;
        }
        auto t = std::make_shared<Tensor>();
        t->shape_ = {k, m};
        t->type_ = ggml_type;
        check(mi_qmm_weight_upload(ctx_, ggml_type, gguf_bytes, k, m, MI_QMM_HOST, &t->weight_));
        tensors_[name] = t;
    }
    // An expert stack [K, M, E] for MulmatID: E matrices of M rows one after the other, GGUF's layout of
    // a 3-D expert tensor (/root/reference/convert/convert_gemma4.go:274-275).
    void LoadExperts(const std::string &name, int ggml_type, int64_t k, int64_t m, int64_t n_expert,
                     const void *gguf_bytes) {
        auto t = std::make_shared<Tensor>();
        t->shape_ = {k, m, n_expert};
        t->type_ = ggml_type;
        check(mi_qmm_weight_upload(ctx_, ggml_type, gguf_bytes, k, m * n_expert, MI_QMM_HOST, &t->weight_));
        tensors_[name] = t;
    }
    // A whole model file (the modelPath ml.NewBackend receives, /root/reference/ml/backend.go:83): every
    // 2-D tensor (and 3-D expert stack) of a type the Mulmat path multiplies is uploaded straight from the file mapping;
    // other tensors (norms, f32 embeddings) are outside this path and are skipped.  Returns how many
    // tensors were loaded.
    int LoadFile(const std::string &path) {
        mi_qmm_gguf *f = nullptr;
        check(mi_qmm_gguf_open(path.c_str(), &f));
        int64_t n = 0;
        int loaded = 0, rc = mi_qmm_gguf_info(f, nullptr, nullptr, nullptr, nullptr, &n);
        for (int64_t i = 0; rc == MI_QMM_OK && i < n; i++) {
            const char *name = nullptr;
            int type = 0, nd = 0;
            int64_t dims[4];
            rc = mi_qmm_gguf_tensor(f, i, &name, &type, &nd, dims, nullptr, nullptr);
            // (Q4_0 / Q8_0 / Q4_K / Q6_K, MXFP4 with rows of whole 256-element steps; F32 / F16 / BF16 / Q5_K matrices and MXFP4 ones kept
            // padded go through mi_qmm_mulmat / mi_qmm_mulmat_id directly, not through this mirror)
            const int q8 = mi_qmm_vec_dot_type(type);
            if (rc != MI_QMM_OK || (nd != 2 && nd != 3) || (q8 != MI_QMM_TYPE_Q8_0 && q8 != MI_QMM_TYPE_Q8_K) || type == MI_QMM_TYPE_Q5_K ||
                ((type == MI_QMM_TYPE_MXFP4 || type == MI_QMM_TYPE_Q5_0) && dims[0] % 256 != 0)) continue;
            auto t = std::make_shared<Tensor>();
            t->shape_.assign(dims, dims + nd);
            t->type_ = type;
            rc = mi_qmm_gguf_upload(ctx_, f, i, &t->weight_);
            if (rc == MI_QMM_OK) { tensors_[name] = t; loaded++; }
        }
        mi_qmm_gguf_close(f);
        check(rc);
        return loaded;
    }
    std::shared_ptr<Tensor> Get(const std::string &name) const {
        auto it = tensors_.find(name);
        return it == tensors_.end() ? nullptr : it->second;  // nil for an unknown name, like the reference
    }
    std::unique_ptr<Context> NewContext();
    void Close() {
        tensors_.clear();
        if (ctx_) mi_qmm_destroy(ctx_);
        ctx_ = nullptr;
    }
    mi_qmm_ctx *handle() const { return ctx_; }

private:
    mi_qmm_ctx *ctx_ = nullptr;
    std::map<std::string, std::shared_ptr<Tensor>> tensors_;
};

class Context {
public:
    explicit Context(Backend &b) : b_(b) {}
    std::shared_ptr<Tensor> FromFloats(const std::vector<float> &s, std::vector<int64_t> shape) {
        int64_t n = 1;
        for (auto d : shape) n *= d;
        if (n != (int64_t)s.size()) throw Error(MI_QMM_ERR_INVALID, "FromFloats: value count does not match the shape");
        auto t = std::make_shared<Tensor>();
        t->shape_ = std::move(shape);
        t->data_ = s;
        t->ready_ = true;
        return t;
    }
    std::shared_ptr<Tensor> FromInts(const std::vector<int32_t> &s, std::vector<int64_t> shape) {
        int64_t n = 1;
        for (auto d : shape) n *= d;
        if (n != (int64_t)s.size()) throw Error(MI_QMM_ERR_INVALID, "FromInts: value count does not match the shape");
        auto t = std::make_shared<Tensor>();
        t->shape_ = std::move(shape);
        t->type_ = 26;  // ggml's int32, /root/reference/fs/ggml/type.go:252-279
        t->ints_ = s;
        t->ready_ = true;
        return t;
    }
    // Run the pending nodes in the order they were recorded.  Mulmat nodes that read the same x are handled
    // together: decode-sized ones (n <= 8) go out four weights at a time through the entry point that
    // quantizes x inside the GEMV launch; larger ones share one quantization of x.  Producer nodes (RMSNorm,
    // SILU) are materialized only when listed in `wanted` or read by something other than a product;
    // otherwise they run inside the quantization of the products that read them.
    void Compute(const std::vector<std::shared_ptr<Tensor>> &wanted = {}) {
        std::set<const Tensor *> needed;
        for (auto &t : wanted) needed.insert(t.get());
        for (auto &n : nodes_) {
            if (n->ready_ || n->absorbed_) continue;
            if (n->prod_) {
                needed.insert(n->prod_src_.get());
                if (n->prod_aux_) needed.insert(n->prod_aux_.get());
                if (n->prod_ == MI_QMM_PRODUCE_SWIGLU && !n->prod_aux_) needed.insert(n.get());  // the bare silu
            }
        }
        // gate.SILU(up) on two pending products of one x that nothing else reads: one call computes the gated
        // result (mi_qmm_mulmat_swiglu), the two products are never materialized
        std::map<const Tensor *, int> n_readers;
        for (auto &n : nodes_) {
            if (n->ready_ || n->absorbed_) continue;
            if (n->prod_) {
                n_readers[n->prod_src_.get()]++;
                if (n->prod_aux_) n_readers[n->prod_aux_.get()]++;
            } else {
                n_readers[n->op_x_.get()]++;
            }
        }
        std::map<const Tensor *, Tensor *> pair_of;
        for (auto &n : nodes_) {
            if (n->ready_ || n->prod_ != MI_QMM_PRODUCE_SWIGLU) continue;
            Tensor *gate = n->prod_src_.get(), *up = n->prod_aux_.get();
            auto pending_product = [&](const Tensor *p) {
                return !p->ready_ && !p->absorbed_ && p->op_w_ && !needed_by_caller(wanted, p) && n_readers[p] == 1;
            };
            if (gate == up || !pending_product(gate) || !pending_product(up) || gate->op_x_ != up->op_x_ ||
                gate->op_ids_ != up->op_ids_ || gate->op_w_->shape_ != up->op_w_->shape_)
                continue;
            // one activation row (one token for expert stacks): the single-launch form; with more rows the gating
            // is better placed in its reader's quantization
            int64_t rows = 1;
            if (gate->op_ids_) rows = gate->op_ids_->Dim(1);
            else for (size_t i = 1; i < gate->op_x_->shape_.size(); i++) rows *= gate->op_x_->shape_[i];
            if (rows != 1) continue;
            pair_of[gate] = pair_of[up] = n.get();
            const Tensor *x = gate->op_x_.get();
            // only a norm in front of plain products runs inside the paired launch
            if (x->prod_ && (x->prod_ != MI_QMM_PRODUCE_RMSNORM || gate->op_ids_)) needed.insert(x);
        }
        for (auto &node : nodes_) {
            Tensor *t = node.get();
            if (t->ready_ || t->absorbed_) continue;
            if (pair_of.count(t)) {
                Tensor *silu = pair_of[t], *gate = silu->prod_src_.get(), *up = silu->prod_aux_.get();
                Tensor *x = gate->op_x_.get();
                if (gate->op_ids_) {
                    const Tensor &ids = *gate->op_ids_;
                    silu->data_.assign((size_t)(gate->op_w_->Dim(1) * ids.Dim(0) * ids.Dim(1)), 0.f);
                    check(mi_qmm_mulmat_id_swiglu(b_.handle(), gate->op_w_->weight_, up->op_w_->weight_, gate->op_w_->Dim(2),
                                                  x->Floats().data(), x->Dim(1), ids.ints_.data(), ids.Dim(0), ids.Dim(1),
                                                  silu->data_.data(), MI_QMM_HOST));
                    silu->ready_ = true;
                    gate->absorbed_ = up->absorbed_ = true;
                    continue;
                }
                const bool norm = !x->ready_ && x->prod_ == MI_QMM_PRODUCE_RMSNORM;
                const Tensor &src = norm ? *x->prod_src_ : *x;
                const int64_t k = src.Dim(0), n = (int64_t)src.Floats().size() / k;
                silu->data_.assign((size_t)(n * gate->Dim(0)), 0.f);
                check(mi_qmm_mulmat_swiglu(b_.handle(), gate->op_w_->weight_, up->op_w_->weight_,
                                           norm ? MI_QMM_PRODUCE_RMSNORM : MI_QMM_PRODUCE_NONE,
                                           norm && x->prod_aux_ ? x->prod_aux_->Floats().data() : nullptr, norm ? x->prod_eps_ : 0.f,
                                           src.data_.data(), n, silu->data_.data(), MI_QMM_HOST));
                silu->ready_ = true;
                gate->absorbed_ = up->absorbed_ = true;
                continue;
            }
            if (t->prod_) {
                if (!needed.count(t)) continue;
                const Tensor &src = *t->prod_src_;
                const int64_t k = src.Dim(0), n = (int64_t)src.Floats().size() / k;
                t->data_.assign(src.data_.size(), 0.f);
                if (t->prod_ == MI_QMM_PRODUCE_RMSNORM)
                    check(mi_qmm_rms_norm(b_.handle(), src.data_.data(), t->prod_aux_ ? t->prod_aux_->Floats().data() : nullptr,
                                          t->prod_eps_, k, n, t->data_.data(), MI_QMM_HOST));
                else
                    check(mi_qmm_swiglu(b_.handle(), src.data_.data(), t->prod_aux_ ? t->prod_aux_->Floats().data() : nullptr, k, n,
                                        t->data_.data(), MI_QMM_HOST));
                t->ready_ = true;
                continue;
            }
            Tensor *x = t->op_x_.get();
            std::vector<Tensor *> group;  // the pending nodes that go out with t
            std::vector<const mi_qmm_weight *> ws;
            std::vector<float *> ys;
            if (t->op_ids_) {
                // expert-indexed nodes that read the same x and ids (gate and up of an expert FFN) go out together
                const Tensor &ids = *t->op_ids_;
                for (auto &u : nodes_)
                    if (!u->ready_ && !u->absorbed_ && !pair_of.count(u.get()) && u->op_ids_ == t->op_ids_ && u->op_x_.get() == x &&
                        u->op_w_->Dim(2) == t->op_w_->Dim(2))
                        group.push_back(u.get());
                for (Tensor *u : group) {
                    u->data_.assign((size_t)(u->op_w_->Dim(1) * ids.Dim(0) * ids.Dim(1)), 0.f);
                    ws.push_back(u->op_w_->weight_);
                    ys.push_back(u->data_.data());
                }
                if (!x->ready_ && x->prod_) {
                    // x is a producer nobody needs in f32 (silu(gate) * up in front of the down experts)
                    for (size_t i = 0; i < ws.size(); i++)
                        check(mi_qmm_mulmat_id_produced(b_.handle(), ws[i], t->op_w_->Dim(2), x->prod_,
                                                        x->prod_aux_ ? x->prod_aux_->Floats().data() : nullptr, x->prod_eps_,
                                                        x->prod_src_->Floats().data(), x->Dim(1), ids.ints_.data(), ids.Dim(0),
                                                        ids.Dim(1), ys[i], MI_QMM_HOST));
                } else {
                    check(mi_qmm_mulmat_id_multi(b_.handle(), ws.data(), (int)ws.size(), t->op_w_->Dim(2), x->Floats().data(),
                                                 x->Dim(1), ids.ints_.data(), ids.Dim(0), ids.Dim(1), ys.data(), MI_QMM_HOST));
                }
                for (Tensor *u : group) u->ready_ = true;
                continue;
            }
            const bool fused = !x->ready_ && x->prod_;  // a producer nobody needs in f32
            const Tensor &src = fused ? *x->prod_src_ : *x;
            const int64_t k = src.Dim(0), n = (int64_t)src.Floats().size() / k;
            for (auto &u : nodes_)
                if (!u->ready_ && !u->absorbed_ && !pair_of.count(u.get()) && !u->prod_ && !u->op_ids_ && u->op_x_.get() == x &&
                    (fused || n > 8 || u->op_w_->type_ == t->op_w_->type_))  // decode launches hold one weight type
                    group.push_back(u.get());
            for (Tensor *u : group) u->data_.assign((size_t)(n * u->Dim(0)), 0.f);
            if (fused) {
                for (Tensor *u : group) { ws.push_back(u->op_w_->weight_); ys.push_back(u->data_.data()); }
                check(mi_qmm_mulmat_produced(b_.handle(), ws.data(), (int)ws.size(), x->prod_,
                                             x->prod_aux_ ? x->prod_aux_->Floats().data() : nullptr, x->prod_eps_,
                                             src.data_.data(), n, ys.data(), MI_QMM_HOST));
            } else if (n <= 8) {
                for (size_t i = 0; i < group.size(); i += 4) {
                    const mi_qmm_weight *w4[4];
                    float *y4[4];
                    int cnt = 0;
                    for (size_t j = i; j < group.size() && j < i + 4; j++, cnt++) {
                        w4[cnt] = group[j]->op_w_->weight_;
                        y4[cnt] = group[j]->data_.data();
                    }
                    check(mi_qmm_mulmat_multi(b_.handle(), w4, cnt, x->data_.data(), n, y4, MI_QMM_HOST));
                }
            } else {
                // one quantization of x per activation format in use
                for (int q8 : {MI_QMM_TYPE_Q8_0, MI_QMM_TYPE_Q8_K}) {
                    std::vector<Tensor *> part;
                    for (Tensor *u : group)
                        if (mi_qmm_vec_dot_type(u->op_w_->type_) == q8) part.push_back(u);
                    if (part.empty()) continue;
                    mi_qmm_act *act = nullptr;
                    check(mi_qmm_act_create(b_.handle(), q8, k, n, &act));
                    int rc = mi_qmm_act_quantize(b_.handle(), act, x->data_.data(), n, MI_QMM_HOST);
                    for (size_t i = 0; rc == MI_QMM_OK && i < part.size(); i++)
                        rc = mi_qmm_mulmat_q8(b_.handle(), part[i]->op_w_->weight_, act, part[i]->data_.data(), MI_QMM_HOST,
                                              MI_QMM_PATH_AUTO);
                    mi_qmm_act_free(act);
                    check(rc);
                }
            }
            for (Tensor *u : group) u->ready_ = true;
        }
    }
    void Close() { nodes_.clear(); }

private:
    friend class Tensor;
    static bool needed_by_caller(const std::vector<std::shared_ptr<Tensor>> &wanted, const Tensor *p) {
        for (auto &t : wanted)
            if (t.get() == p) return true;
        return false;
    }
    Backend &b_;
    std::vector<std::shared_ptr<Tensor>> nodes_;
};

inline std::unique_ptr<Context> Backend::NewContext() { return std::unique_ptr<Context>(new Context(*this)); }

inline std::shared_ptr<Tensor> Tensor::Mulmat(Context &ctx, const std::shared_ptr<Tensor> &t2) {
    if (!weight_) throw Error(MI_QMM_ERR_INVALID, "Mulmat: the receiver must be a quantized weight from Backend::Get");
    if (shape_.size() != 2) throw Error(MI_QMM_ERR_INVALID, "Mulmat: the weight must be 2-D (expert stacks go through MulmatID)");
    if (!t2 || t2->type_ != MI_QMM_TYPE_F32) throw Error(MI_QMM_ERR_INVALID, "Mulmat: activations must be f32");
    if (t2->Dim(0) != Dim(0)) throw Error(MI_QMM_ERR_INVALID, "Mulmat: inner dimensions differ");
    auto out = std::make_shared<Tensor>();
    out->shape_ = {shape_[1]};
    for (size_t i = 1; i < t2->shape_.size(); i++) out->shape_.push_back(t2->shape_[i]);
    out->op_w_ = this;
    out->op_x_ = t2;
    ctx.nodes_.push_back(out);
    return out;
}

inline std::shared_ptr<Tensor> Tensor::MulmatID(Context &ctx, const std::shared_ptr<Tensor> &t2,
                                                const std::shared_ptr<Tensor> &ids) {
    if (!weight_ || shape_.size() != 3)
        throw Error(MI_QMM_ERR_INVALID, "MulmatID: the receiver must be a 3-D quantized expert stack from Backend::Get");
    if (!t2 || t2->type_ != MI_QMM_TYPE_F32 || !ids || ids->type_ != 26)
        throw Error(MI_QMM_ERR_INVALID, "MulmatID: activations must be f32 and ids int32");
    if (t2->Dim(0) != Dim(0)) throw Error(MI_QMM_ERR_INVALID, "MulmatID: inner dimensions differ");
    if (ids->shape_.size() > 2 || t2->shape_.size() > 3 || ids->Dim(1) != t2->Dim(2))
        throw Error(MI_QMM_ERR_INVALID, "MulmatID: ids and activations disagree on the token count");
    auto out = std::make_shared<Tensor>();
    out->shape_ = {shape_[1], ids->Dim(0), ids->Dim(1)};
    out->op_w_ = this;
    out->op_x_ = t2;
    out->op_ids_ = ids;
    ctx.nodes_.push_back(out);
    return out;
}

inline std::shared_ptr<Tensor> Tensor::RMSNorm(Context &ctx, const std::shared_ptr<Tensor> &weight, float eps) {
    if (type_ != MI_QMM_TYPE_F32 || weight_ || (weight && (weight->type_ != MI_QMM_TYPE_F32 || weight->weight_)))
        throw Error(MI_QMM_ERR_INVALID, "RMSNorm: operands must be f32");
    if (weight && (!weight->ready_ || (int64_t)weight->data_.size() != Dim(0)))
        throw Error(MI_QMM_ERR_INVALID, "RMSNorm: the weight must hold one value per element of dimension 0");
    auto out = std::make_shared<Tensor>();
    out->shape_ = shape_;
    out->prod_ = MI_QMM_PRODUCE_RMSNORM;
    out->prod_src_ = shared_from_this();
    out->prod_aux_ = weight;
    out->prod_eps_ = eps;
    ctx.nodes_.push_back(out);
    return out;
}

inline std::shared_ptr<Tensor> Tensor::SILU(Context &ctx, const std::shared_ptr<Tensor> &up) {
    // up == nullptr: the bare activation silu(self), always an f32 node of its own
    if (type_ != MI_QMM_TYPE_F32 || weight_ || (up && (up->type_ != MI_QMM_TYPE_F32 || up->weight_ || shape_ != up->shape_)))
        throw Error(MI_QMM_ERR_INVALID, "SILU: gate and up must be f32 of one shape");
    auto out = std::make_shared<Tensor>();
    out->shape_ = shape_;
    out->prod_ = MI_QMM_PRODUCE_SWIGLU;
    out->prod_src_ = shared_from_this();
    out->prod_aux_ = up;
    ctx.nodes_.push_back(out);
    return out;
}

}  // namespace ollama_amd
