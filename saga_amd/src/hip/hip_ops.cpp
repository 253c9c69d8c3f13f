// Node lowerings and graph transforms of the hip engine: every node type of the front end
// becomes a short list of kernel-library calls (saga_hip.h), forward and backward.
// Role of the reference's src/cuda/cuda_dnn.cpp; cited per lowering.
#include <math.h>

#include "hip_common.hpp"

namespace saga {

namespace {

using T = std::shared_ptr<HipTensor>;

saga_stream_t S(HipProgram &p) { return (saga_stream_t)p.m_ctx->m_stream; }

double nbytes(const T &t) { return (double)t->m_dims.elements() * Tensor::DataTypeSize(t->m_data_type); }

// 2 * N * K * P * Q * (C / group) * R * S for a convolution with input x, filter w, output y
double conv_flops(const T &x, const T &w, const T &y, int group)
{
    return 2.0 * (double)y->m_dims.elements() * (double)((int)w->m_dims[1]) * (int)w->m_dims[2] * (int)w->m_dims[3];
}

T alias_of(const T &base, const Dims &dims, const std::vector<int64_t> &strides, int64_t offset,
           const std::optional<const std::string> &name)
{
    return std::make_shared<HipTensor>(base->m_storage, dims, strides, offset, name);
}

// ---------------------------------------------------------------- convolution
// reference: src/cuda/cuda_dnn.cpp:323-577

struct ConvDesc {
    SagaConvParams params;
};

// Per-channel partial sums of a convolution's output, handed from the ConvFwd that produces
// them in its epilogue to the BnTrain that would otherwise read the tensor once more.
struct ConvStatsLink {
    std::shared_ptr<HipMemory> partial;
    int rows = 0;
    bool valid = false; // set by every ConvFwd::exec, consumed by the BnTrain::exec that follows
};

struct ConvFwd : public HipOperation {
    const T x_, w_, y_;
    const SagaConvParams cp_;
    float beta_ = 0;
    std::shared_ptr<ConvStatsLink> stats_;
    // inference: the batch norm that consumes y (with its residual and relu) runs in the epilogue
    // and the result goes straight to the norm's output
    T bn_s_, bn_b_, bn_m_, bn_v_, bn_z_, bn_y_;
    float bn_eps_ = 0;
    int bn_flags_ = 0;
    ConvFwd(HipProgram &p, T x, T w, T y, SagaConvParams cp) : HipOperation("convfwd"), x_(x), w_(w), y_(y), cp_(cp)
    {
        const SagaTensorView vx = x->shapeView(), vw = w->shapeView(), vy = y->shapeView();
        p.m_ctx->m_workspace.request(saga_hip_conv2d_workspace_size(SAGA_CONV_FWD, &vx, &vw, &vy, &cp_));
    }
    // called by a batch normalisation that consumes y; nullptr if this convolution cannot supply them
    std::shared_ptr<ConvStatsLink> offerStats()
    {
        if(stats_)
            return stats_;
        const SagaTensorView vx = x_->shapeView(), vw = w_->shapeView(), vy = y_->shapeView();
        const size_t bytes = saga_hip_conv2d_fwd_bnstats_size(&vx, &vw, &vy, &cp_);
        if(!bytes)
            return nullptr;
        stats_ = std::make_shared<ConvStatsLink>();
        stats_->partial = std::make_shared<HipMemory>(bytes);
        return stats_;
    }
    bool foldBn(T s, T b, T m, T v, T z, T y, float eps, int flags)
    {
        if(stats_ || bn_y_ || x_->m_data_type != Tensor::DataType::HALF)
            return false;
        bn_s_ = s; bn_b_ = b; bn_m_ = m; bn_v_ = v; bn_z_ = z; bn_y_ = y;
        bn_eps_ = eps;
        bn_flags_ = flags;
        m_kind = "convfwd.bn";
        return true;
    }
    void execFolded(HipProgram &p)
    {
        const SagaTensorView vx = x_->view(), vw = w_->view(), vo = bn_y_->view();
        SagaTensorView vz;
        if(bn_z_)
            vz = bn_z_->view();
        const float *s = (const float *)bn_s_->deviceMem(), *b = (const float *)bn_b_->deviceMem();
        const float *m = (const float *)bn_m_->deviceMem(), *v = (const float *)bn_v_->deviceMem();
        const int r = saga_hip_conv2d_fwd_bn_infer(&vx, &vw, &vo, bn_z_ ? &vz : nullptr, &cp_, s, b, m, v, bn_eps_, bn_flags_,
                                                   p.m_ctx->m_workspace.ptr(), p.m_ctx->m_workspace.size(), S(p));
        if(r == 0)
            return;
        if(r != SAGA_HIP_EUNSUPPORTED)
            chkSaga(r);
        // two passes through the convolution's own output tensor
        const SagaTensorView vy = y_->view();
        chkSaga(saga_hip_conv2d_fwd(&vx, &vw, &vy, &cp_, 1.0f, 0.0f, p.m_ctx->m_workspace.ptr(),
                                    p.m_ctx->m_workspace.size(), S(p)));
        chkSaga(saga_hip_bn_infer(&vy, bn_z_ ? &vz : nullptr, &vo, s, b, m, v, bn_eps_, bn_flags_, S(p)));
    }
    void exec(HipProgram &p) override
    {
        if(bn_y_)
            return execFolded(p);
        const SagaTensorView vx = x_->view(), vw = w_->view(), vy = y_->view();
        if(stats_) {
            stats_->valid = false;
            if(beta_ == 0.0f) {
                const int r = saga_hip_conv2d_fwd_bnstats(&vx, &vw, &vy, &cp_, 1.0f, p.m_ctx->m_workspace.ptr(),
                                                          p.m_ctx->m_workspace.size(), (float *)stats_->partial->m_ptr,
                                                          stats_->partial->m_bytes, &stats_->rows, S(p));
                if(r == 0) {
                    stats_->valid = true;
                    return;
                }
                if(r != SAGA_HIP_EUNSUPPORTED)
                    chkSaga(r);
            }
        }
        chkSaga(saga_hip_conv2d_fwd(&vx, &vw, &vy, &cp_, 1.0f, beta_, p.m_ctx->m_workspace.ptr(),
                                    p.m_ctx->m_workspace.size(), S(p)));
    }
    HipOpArgs listInputs() const override
    {
        HipOpArgs r{{"x", x_}, {"w", w_}};
        if(bn_y_) {
            r.insert(r.end(), {{"s", bn_s_}, {"b", bn_b_}, {"m", bn_m_}, {"v", bn_v_}});
            if(bn_z_)
                r.push_back({"z", bn_z_});
        }
        return r;
    }
    HipOpArgs listOutputs() const override { return {{"y", bn_y_ ? bn_y_ : y_}}; }
    float *getBeta(const T &t) override { return !bn_y_ && t == y_ ? &beta_ : nullptr; }
    double flops() const override { return conv_flops(x_, w_, y_, cp_.group); }
    double bytes() const override
    {
        return nbytes(x_) + nbytes(w_) + nbytes(y_) * (beta_ != 0 ? 2 : 1) + (bn_z_ ? nbytes(bn_z_) : 0);
    }
};

// The fp16 channels-last backward-data kernel reads the filter as C,R,S,K.  Instead of one small transpose
// launch per layer and step, every backward-data operation of a program registers its filter here, and this
// one operation - placed in the forward list, i.e. after the previous step's optimizer and before any
// backward operation - transposes them all in a single launch into per-layer tensors.
struct FilterTransposeBatch : public HipOperation {
    struct Item {
        T w, wt;
    };
    std::vector<Item> items_;
    std::unique_ptr<HipMemory> jobs_dev_;
    std::vector<SagaFilterTransposeJob> jobs_;
    uint64_t epoch_ = ~(uint64_t)0;
    int total_blocks_ = 0;
    bool dirty_ = true;
    FilterTransposeBatch() : HipOperation("filtertranspose") {}
    void add(T w, T wt)
    {
        items_.push_back({w, wt});
        dirty_ = true;
    }
    void exec(HipProgram &p) override
    {
        if(items_.empty())
            return;
        if(dirty_ || epoch_ != p.m_ctx->m_mem_epoch) { // a storage moved: the job table holds addresses
            jobs_.clear();
            total_blocks_ = 0;
            for(auto &it : items_) {
                const SagaTensorView vw = it.w->view();
                SagaFilterTransposeJob j;
                j.w = it.w->deviceMem();
                j.wt = it.wt->deviceMem();
                j.K = vw.dims[0];
                j.C = vw.dims[1];
                j.RS = vw.dims[2] * vw.dims[3];
                j.first_block = total_blocks_;
                total_blocks_ += saga_hip_filter_transpose_blocks(&vw);
                jobs_.push_back(j);
            }
            const size_t bytes = jobs_.size() * sizeof(SagaFilterTransposeJob);
            if(!jobs_dev_ || jobs_dev_->m_bytes < bytes)
                jobs_dev_ = std::make_unique<HipMemory>(bytes);
            // synchronous copy of a few kilobytes, only when the table changed; jobs_ stays valid meanwhile
            chkHip(hipStreamSynchronize(p.m_ctx->m_stream));
            chkHip(hipMemcpy(jobs_dev_->m_ptr, jobs_.data(), bytes, hipMemcpyHostToDevice));
            epoch_ = p.m_ctx->m_mem_epoch;
            dirty_ = false;
        }
        chkSaga(saga_hip_filter_transpose_batched((const SagaFilterTransposeJob *)jobs_dev_->m_ptr, (int)jobs_.size(),
                                                  total_blocks_, S(p)));
    }
    HipOpArgs listInputs() const override
    {
        HipOpArgs r;
        for(auto &it : items_)
            r.push_back({"w", it.w});
        return r;
    }
    HipOpArgs listOutputs() const override
    {
        HipOpArgs r;
        for(auto &it : items_)
            r.push_back({"wt", it.wt});
        return r;
    }
    bool killOutput(const std::shared_ptr<HipStorage> &s) override
    {
        for(size_t i = 0; i < items_.size(); i++)
            if(items_[i].wt->m_storage == s) {
                items_.erase(items_.begin() + i);
                dirty_ = true;
                return true;
            }
        return false;
    }
    // the table upload synchronises; keep the operation out of recorded graphs
    bool graphSafe() const override { return false; }
    double bytes() const override
    {
        double b = 0;
        for(auto &it : items_)
            b += 2.0 * nbytes(it.w);
        return b;
    }
};

// Per-channel sums of a relu-masked gradient, handed from the ConvBwdData that is the last writer of a
// batch norm's output gradient to that norm's BnBwd, which then skips its own first pass over the tensor.
struct BnBwdLinkState {
    std::shared_ptr<HipMemory> partial;
    int rows = 0;
    bool valid = false; // set by every ConvBwdData::exec, consumed by the BnBwd::exec that follows
    // the kernel library refused the linked launch (the norm's input is a view it cannot read in the epilogue):
    // both operations stay on their separate paths from then on and report the traffic of those
    bool refused = false;
};

struct ConvBwdData : public HipOperation {
    const T w_, dy_, dx_;
    T wt_; // the filter as C,R,S,K, written by the program's FilterTransposeBatch (null: transposed per call)
    const SagaConvParams cp_;
    float beta_ = 0;
    // dx is the gradient of a batch norm's (+ relu) output and this is its last writer: the epilogue masks it
    // and leaves the sums of the norm's backward (x, scale, bias, saved mean and 1/std of that norm)
    std::shared_ptr<BnBwdLinkState> link_;
    T bn_x_, bn_s_, bn_b_, bn_sm_, bn_sv_;
    int bn_flags_ = 0;
    std::shared_ptr<BnBwdLinkState> linkBnBwd(T x, T s, T b, T sm, T sv, int flags)
    {
        if(link_)
            return nullptr;
        // The epilogue's extra work (one more tensor to read, the mask and the sums) costs the convolution
        // more than the norm's first pass saves where the convolution has little arithmetic per output to
        // hide it behind: measured on MI355X at batch 256, linking loses at 64 channels (1x1 and 3x3) and
        // at 128 channels under a 1x1 filter, and wins from there up.  SAGA_HIP_BNBWD_LINK_ALL links all.
        const int channels = (int)dx_->m_dims[1], taps = (int)w_->m_dims[2] * (int)w_->m_dims[3];
        if(!(channels >= 256 || (channels >= 128 && taps > 1)) && !getenv("SAGA_HIP_BNBWD_LINK_ALL"))
            return nullptr;
        const SagaTensorView vx = dx_->shapeView(), vw = w_->shapeView(), vy = dy_->shapeView();
        const size_t bytes = saga_hip_conv2d_bwd_data_bnbwd_size(&vy, &vw, &vx, &cp_);
        if(!bytes)
            return nullptr;
        link_ = std::make_shared<BnBwdLinkState>();
        link_->partial = std::make_shared<HipMemory>(bytes);
        bn_x_ = x; bn_s_ = s; bn_b_ = b; bn_sm_ = sm; bn_sv_ = sv;
        bn_flags_ = flags;
        m_kind = "convbwddata.bn";
        return link_;
    }
    ConvBwdData(HipProgram &p, HipProgramUnit &pu, T w, T dy, T dx, SagaConvParams cp)
      : HipOperation("convbwddata"), w_(w), dy_(dy), dx_(dx), cp_(cp)
    {
        const SagaTensorView vx = dx->shapeView(), vw = w->shapeView(), vy = dy->shapeView();
        p.m_ctx->m_workspace.request(saga_hip_conv2d_workspace_size(SAGA_CONV_BWD_DATA, &vx, &vw, &vy, &cp_));
        const size_t wt_bytes = saga_hip_conv2d_bwd_data_wt_bytes(&vy, &vw, &vx, &cp_);
        if(wt_bytes && !getenv("SAGA_HIP_NO_BATCHED_TRANSPOSE")) {
            wt_ = std::make_shared<HipTensor>(Tensor::DataType::HALF, Dims{(int64_t)(wt_bytes / 2)}, HipLayout::NCHW,
                                              p.m_ctx.get(), w->namePostfix("transposed"));
            if(!p.m_transpose_batch) {
                p.m_transpose_batch = std::make_shared<FilterTransposeBatch>();
                pu.fwd(p.m_transpose_batch);
            }
            static_cast<FilterTransposeBatch *>(p.m_transpose_batch.get())->add(w, wt_);
        }
    }
    void exec(HipProgram &p) override
    {
        const SagaTensorView vdy = dy_->view(), vw = w_->view(), vdx = dx_->view();
        if(link_ && !link_->refused) {
            link_->valid = false;
            const SagaTensorView vx = bn_x_->view();
            SagaBnBwdLink l = {&vx,
                               (const float *)bn_s_->deviceMem(),
                               (const float *)bn_b_->deviceMem(),
                               (const float *)bn_sm_->deviceMem(),
                               (const float *)bn_sv_->deviceMem(),
                               bn_flags_,
                               0,
                               (float *)link_->partial->m_ptr,
                               link_->partial->m_bytes};
            const int r = saga_hip_conv2d_bwd_data_bnbwd(&vdy, &vw, wt_ ? wt_->deviceMem() : nullptr, &vdx, &cp_, 1.0f, beta_,
                                                         p.m_ctx->m_workspace.ptr(), p.m_ctx->m_workspace.size(), &l, S(p));
            if(r == 0) {
                link_->rows = l.partial_rows;
                link_->valid = true;
                return;
            }
            if(r != SAGA_HIP_EUNSUPPORTED)
                chkSaga(r);
            link_->refused = true;
        }
        chkSaga(saga_hip_conv2d_bwd_data_wt(&vdy, &vw, wt_ ? wt_->deviceMem() : nullptr, &vdx, &cp_, 1.0f, beta_,
                                            p.m_ctx->m_workspace.ptr(), p.m_ctx->m_workspace.size(), S(p)));
    }
    HipOpArgs listInputs() const override
    {
        HipOpArgs r{{"w", w_}, {"dy", dy_}};
        if(wt_)
            r.push_back({"wt", wt_});
        if(link_)
            r.insert(r.end(), {{"bn.x", bn_x_}, {"bn.s", bn_s_}, {"bn.b", bn_b_}, {"bn.sm", bn_sm_}, {"bn.sv", bn_sv_}});
        return r;
    }
    HipOpArgs listOutputs() const override { return {{"dx", dx_}}; }
    float *getBeta(const T &t) override { return t == dx_ ? &beta_ : nullptr; }
    double flops() const override { return conv_flops(dx_, w_, dy_, cp_.group); }
    double bytes() const override
    {
        return nbytes(dy_) + nbytes(w_) + nbytes(dx_) * ((beta_ != 0 ? 2 : 1) + (link_ && !link_->refused ? 1 : 0));
    }
};

struct ConvBwdFilter : public HipOperation {
    const T x_, dy_, dw_;
    const SagaConvParams cp_;
    float beta_ = 0;
    ConvBwdFilter(HipProgram &p, T x, T dy, T dw, SagaConvParams cp)
      : HipOperation("convbwdfilter"), x_(x), dy_(dy), dw_(dw), cp_(cp)
    {
        const SagaTensorView vx = x->shapeView(), vw = dw->shapeView(), vy = dy->shapeView();
        p.m_ctx->m_workspace.request(saga_hip_conv2d_workspace_size(SAGA_CONV_BWD_FILTER, &vx, &vw, &vy, &cp_));
    }
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view(), vdy = dy_->view(), vdw = dw_->view();
        chkSaga(saga_hip_conv2d_bwd_filter(&vx, &vdy, &vdw, &cp_, 1.0f, beta_, p.m_ctx->m_workspace.ptr(),
                                           p.m_ctx->m_workspace.size(), S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", x_}, {"dy", dy_}}; }
    HipOpArgs listOutputs() const override { return {{"dw", dw_}}; }
    float *getBeta(const T &t) override { return t == dw_ ? &beta_ : nullptr; }
    double flops() const override { return conv_flops(x_, dw_, dy_, cp_.group); }
    double bytes() const override { return nbytes(x_) + nbytes(dy_) + nbytes(dw_); }
};

// y += b, b broadcast over the channel axis (reference: CudnnAddTensor, :39-68)
struct BiasAdd : public HipOperation {
    const T b_, y_;
    BiasAdd(T b, T y) : HipOperation("biasadd"), b_(b), y_(y) {}
    void exec(HipProgram &p) override
    {
        const SagaTensorView vy = y_->view(), vb = b_->view();
        chkSaga(saga_hip_bias_add(&vy, &vb, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"b", b_}, {"y", y_}}; }
    HipOpArgs listOutputs() const override { return {{"y", y_}}; }
    double bytes() const override { return 2 * nbytes(y_); }
    // the output is read as well as written; report it as accumulating so that liveness sees the read
    float one_ = 1.0f;
    float *getBeta(const T &t) override { return t == y_ ? &one_ : nullptr; }
};

struct BiasBwd : public HipOperation {
    const T dy_, db_;
    float beta_ = 0;
    BiasBwd(HipProgram &p, T dy, T db) : HipOperation("biasbwd"), dy_(dy), db_(db)
    {
        const SagaTensorView vdy = dy->shapeView();
        p.m_ctx->m_workspace.request(saga_hip_bias_bwd_workspace_size(&vdy));
    }
    void exec(HipProgram &p) override
    {
        const SagaTensorView vdy = dy_->view(), vdb = db_->view();
        chkSaga(saga_hip_bias_bwd(&vdy, &vdb, beta_, p.m_ctx->m_workspace.ptr(), p.m_ctx->m_workspace.size(), S(p)));
    }
    HipOpArgs listInputs() const override { return {{"dy", dy_}}; }
    HipOpArgs listOutputs() const override { return {{"db", db_}}; }
    double bytes() const override { return nbytes(dy_); }
    float *getBeta(const T &t) override { return t == db_ ? &beta_ : nullptr; }
};

void conv_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    auto x = p.lower(pu, n.m_inputs["x"]);
    auto y = p.lower(pu, n.m_outputs["y"]);
    auto w = p.lower(pu, n.m_inputs["w"]);
    auto b = n.m_inputs.has("b") ? p.lower(pu, n.m_inputs["b"], y->m_dims.size()) : nullptr;

    SagaConvParams cp;
    cp.pad = n.m_attributes.get("pad", 0);
    cp.stride = n.m_attributes.get("stride", 1);
    cp.dilation = 1; // like the reference backend, which ignores the attribute (:227-231)
    cp.group = n.m_attributes.get("group", 1);
    const bool transpose = n.m_attributes.get("transpose", false);
    const bool training = p.m_pt == ProgramType::TRAINING;

    if(!transpose) {
        pu.fwd(std::make_shared<ConvFwd>(p, x, w, y, cp));
        if(b)
            pu.fwd(std::make_shared<BiasAdd>(b, y));
        if(!training)
            return;
        auto dy = p.lowerGrad(pu, n.m_outputs["y"]);
        if(b) {
            auto db = p.lowerGrad(pu, n.m_inputs["b"], y->m_dims.size());
            pu.bwd(std::make_shared<BiasBwd>(p, dy, db));
            p.upd(n.m_inputs["b"], b, db);
        }
        auto dw = p.lowerGrad(pu, n.m_inputs["w"]);
        pu.bwd(std::make_shared<ConvBwdFilter>(p, x, dy, dw, cp));
        p.upd(n.m_inputs["w"], w, dw);
        if(auto dx = p.lowerGrad(pu, n.m_inputs["x"]))
            pu.bwd(std::make_shared<ConvBwdData>(p, pu, w, dy, dx, cp));
    } else {
        // transposed convolution: the three kernels with x and y exchanged (:542-574)
        pu.fwd(std::make_shared<ConvBwdData>(p, pu, w, x, y, cp));
        if(b)
            pu.fwd(std::make_shared<BiasAdd>(b, y));
        if(!training)
            return;
        auto dy = p.lowerGrad(pu, n.m_outputs["y"]);
        if(b) {
            auto db = p.lowerGrad(pu, n.m_inputs["b"], y->m_dims.size());
            pu.bwd(std::make_shared<BiasBwd>(p, dy, db));
            p.upd(n.m_inputs["b"], b, db);
        }
        auto dw = p.lowerGrad(pu, n.m_inputs["w"]);
        pu.bwd(std::make_shared<ConvBwdFilter>(p, dy, x, dw, cp));
        p.upd(n.m_inputs["w"], w, dw);
        if(auto dx = p.lowerGrad(pu, n.m_inputs["x"]))
            pu.bwd(std::make_shared<ConvFwd>(p, dy, w, dx, cp));
    }
}
REGISTER_HIP_OP("conv", conv_setup);

// ---------------------------------------------------------------- activations
// reference: src/cuda/cuda_dnn.cpp:610-806

struct ActFwd : public HipOperation {
    const T x_, y_;
    const int mode_;
    const float alpha_;
    float beta_ = 0;
    ActFwd(T x, T y, int mode, float alpha) : HipOperation("actfwd"), x_(x), y_(y), mode_(mode), alpha_(alpha) {}
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view(), vy = y_->view();
        chkSaga(saga_hip_act_fwd(mode_, alpha_, &vx, &vy, beta_, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", x_}}; }
    HipOpArgs listOutputs() const override { return {{"y", y_}}; }
    float *getBeta(const T &t) override { return t == y_ ? &beta_ : nullptr; }
    double bytes() const override { return 2 * nbytes(x_); }
    std::string info() const override
    {
        static const char *names[] = {"relu", "sigmoid", "tanh", "swish", "leakyrelu"};
        return names[mode_];
    }
};

struct ActBwd : public HipOperation {
    const T x_, y_, dx_, dy_;
    const int mode_;
    const float alpha_;
    float beta_ = 0;
    ActBwd(T x, T y, T dx, T dy, int mode, float alpha)
      : HipOperation("actbwd"), x_(x), y_(y), dx_(dx), dy_(dy), mode_(mode), alpha_(alpha)
    {
    }
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view(), vy = y_->view(), vdy = dy_->view(), vdx = dx_->view();
        chkSaga(saga_hip_act_bwd(mode_, alpha_, &vx, &vy, &vdy, &vdx, beta_, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", x_}, {"y", y_}, {"dy", dy_}}; }
    HipOpArgs listOutputs() const override { return {{"dx", dx_}}; }
    float *getBeta(const T &t) override { return t == dx_ ? &beta_ : nullptr; }
    double bytes() const override { return (beta_ != 0 ? 4 : 3) * nbytes(dx_); }
};

void activation_setup(HipProgram &p, HipProgramUnit &pu, const Node &n, int mode, float alpha)
{
    auto x = p.lower(pu, n.m_inputs["x"]);
    auto y = p.lowerLike(pu, n.m_outputs["y"], *x);
    pu.fwd(std::make_shared<ActFwd>(x, y, mode, alpha));
    if(p.m_pt == ProgramType::INFERENCE)
        return;
    auto dx = p.lowerGrad(pu, n.m_inputs["x"]);
    auto dy = p.lowerGrad(pu, n.m_outputs["y"]);
    pu.bwd(std::make_shared<ActBwd>(x, y, dx, dy, mode, alpha));
}

void relu_setup(HipProgram &p, HipProgramUnit &pu, const Node &n) { activation_setup(p, pu, n, SAGA_ACT_RELU, 0); }
void sigmoid_setup(HipProgram &p, HipProgramUnit &pu, const Node &n) { activation_setup(p, pu, n, SAGA_ACT_SIGMOID, 0); }
void tanh_setup(HipProgram &p, HipProgramUnit &pu, const Node &n) { activation_setup(p, pu, n, SAGA_ACT_TANH, 0); }
void swish_setup(HipProgram &p, HipProgramUnit &pu, const Node &n) { activation_setup(p, pu, n, SAGA_ACT_SWISH, 0); }
void leakyrelu_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    activation_setup(p, pu, n, SAGA_ACT_LEAKYRELU, n.m_attributes.get("alpha", 0.01f));
}
REGISTER_HIP_OP("relu", relu_setup);
REGISTER_HIP_OP("elu", relu_setup); // the reference registers relu for "elu" as well (:732)
REGISTER_HIP_OP("sigmoid", sigmoid_setup);
REGISTER_HIP_OP("tanh", tanh_setup);
REGISTER_HIP_OP("swish", swish_setup);
REGISTER_HIP_OP("leakyrelu", leakyrelu_setup);

// ---------------------------------------------------------------- fully connected
// reference: src/cuda/cuda_dnn.cpp:968-1130 (column-major cuBLAS calls restated row-major)

struct Gemm : public HipOperation {
    const int ta_, tb_, m_, n_, k_;
    const T a_, b_, c_;
    const int lda_, ldb_, ldc_;
    float beta_ = 0;
    Gemm(int ta, int tb, int m, int n, int k, T a, int lda, T b, int ldb, T c, int ldc, const char *name)
      : HipOperation(name), ta_(ta), tb_(tb), m_(m), n_(n), k_(k), a_(a), b_(b), c_(c), lda_(lda), ldb_(ldb), ldc_(ldc)
    {
        if(a->m_data_type != b->m_data_type || a->m_data_type != c->m_data_type)
            throw std::runtime_error("fc: operand data types differ");
        if(!a->rowMajor() || !b->rowMajor() || !c->rowMajor())
            throw std::runtime_error("fc: operands must be row-major matrices");
    }
    void exec(HipProgram &p) override
    {
        chkSaga(saga_hip_gemm(ta_, tb_, m_, n_, k_, 1.0f, a_->deviceMem(), lda_, b_->deviceMem(), ldb_, beta_,
                              c_->deviceMem(), ldc_, (int)a_->m_data_type, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"a", a_}, {"b", b_}}; }
    HipOpArgs listOutputs() const override { return {{"c", c_}}; }
    float *getBeta(const T &t) override { return t == c_ ? &beta_ : nullptr; }
    double flops() const override { return 2.0 * m_ * n_ * k_; }
    double bytes() const override { return nbytes(a_) + nbytes(b_) + nbytes(c_); }
};

void fc_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    auto x = p.lower(pu, n.m_inputs["x"]);
    auto y = p.lower(pu, n.m_outputs["y"]);
    auto w = p.lower(pu, n.m_inputs["w"]);
    auto b = n.m_inputs.has("b") ? p.lower(pu, n.m_inputs["b"], 2) : nullptr;
    const bool transW = n.m_attributes.get("transW", false);
    const int in = x->m_dims[1], out = y->m_dims[1], batch = x->m_dims[0];

    // y[batch,out] = x[batch,in] * W ; W stored [in,out], or [out,in] when transW
    pu.fwd(std::make_shared<Gemm>(0, transW ? 1 : 0, batch, out, in, x, in, w, transW ? in : out, y, out,
                                  transW ? "fc.fwd.t" : "fc.fwd.n"));
    if(b)
        pu.fwd(std::make_shared<BiasAdd>(b, y));
    if(p.m_pt == ProgramType::INFERENCE)
        return;

    auto dx = p.lowerGrad(pu, n.m_inputs["x"]);
    auto dy = p.lowerGrad(pu, n.m_outputs["y"]);
    auto dw = p.lowerGrad(pu, n.m_inputs["w"]);
    if(transW) // dW[out,in] = dy^T x
        pu.bwd(std::make_shared<Gemm>(1, 0, out, in, batch, dy, out, x, in, dw, in, "fc.bwd.weights.t"));
    else // dW[in,out] = x^T dy
        pu.bwd(std::make_shared<Gemm>(1, 0, in, out, batch, x, in, dy, out, dw, out, "fc.bwd.weights.n"));
    p.upd(n.m_inputs["w"], w, dw);
    if(b) {
        auto db = p.lowerGrad(pu, n.m_inputs["b"], 2);
        pu.bwd(std::make_shared<BiasBwd>(p, dy, db)); // column sums of dy
        p.upd(n.m_inputs["b"], b, db);
    }
    if(dx) // dx[batch,in] = dy * W^T
        pu.bwd(std::make_shared<Gemm>(0, transW ? 0 : 1, batch, in, out, dy, out, w, transW ? in : out, dx, in,
                                      transW ? "fc.bwd.data.t" : "fc.bwd.data.n"));
}
REGISTER_HIP_OP("fc", fc_setup);

// ---------------------------------------------------------------- convert
// reference: src/cuda/cuda_dnn.cpp:1134-1241

struct Convert : public HipOperation {
    const T x_, y_;
    const float scale_;
    Convert(T x, T y, float scale) : HipOperation("convert"), x_(x), y_(y), scale_(scale) {}
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view(), vy = y_->view();
        chkSaga(saga_hip_convert(&vx, &vy, scale_, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", x_}}; }
    HipOpArgs listOutputs() const override { return {{"y", y_}}; }
};

void convert_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    const float scale = n.m_attributes.get("scale", 1.0f);
    auto xh = n.m_inputs["x"], yh = n.m_outputs["y"];
    auto x = p.lower(pu, xh);
    if(xh->m_data_type == yh->m_data_type && scale == 1.0f) {
        p.m_ctx->m_tensors[yh] = alias_of(x, x->m_dims, x->m_strides, x->m_offset, xh->namePostfix("nop-convert"));
        return;
    }
    // the output takes the layout the program would give its type (fp16 -> channels-last)
    auto y = p.lower(pu, yh);
    pu.fwd(std::make_shared<Convert>(x, y, scale));
}
REGISTER_HIP_OP("convert", convert_setup);

Nodes convert_transform(HipProgram &, HipProgramUnit &, const Nodes &input)
{
    Nodes nodes = input;
    bool again = true;
    while(again) {
        again = false;
        for(auto &n : nodes) {
            if(n->m_type != "convert")
                continue;
            auto it = nodes.findSingleDownStreamNode(n->y(), "convert");
            if(it == nodes.end())
                continue;
            auto b = *it;
            auto fused = std::make_shared<Node>("convert");
            fused->m_inputs["x"] = n->m_inputs["x"];
            fused->m_outputs["y"] = b->m_outputs["y"];
            fused->m_attributes["scale"] = n->m_attributes.get("scale", 1.0f) * b->m_attributes.get("scale", 1.0f);
            fused->m_attributes["datatype"] = b->m_attributes.get("datatype", (int)b->y()->m_data_type);
            n = fused;
            nodes.erase(it);
            again = true;
            break;
        }
    }
    return nodes;
}
REGISTER_HIP_TRANSFORM(200, ProgramType::INFERENCE | ProgramType::TRAINING, convert_transform);

// ---------------------------------------------------------------- classifier head
// reference: src/cuda/cuda_dnn.cpp:1244-1355

struct CatClassifierFwd : public HipOperation {
    const T x_, y_;
    CatClassifierFwd(T x, T y) : HipOperation("catclassifierfwd"), x_(x), y_(y) {}
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view();
        chkSaga(saga_hip_catclassifier_fwd(&vx, (int32_t *)y_->deviceMem(), S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", x_}}; }
    HipOpArgs listOutputs() const override { return {{"y", y_}}; }
    double bytes() const override { return nbytes(x_); }
};

struct CatClassifierBwd : public HipOperation {
    const T x_, y_, dx_, dy_;
    T loss_;
    CatClassifierBwd(T x, T y, T dx, T dy, T loss)
      : HipOperation("catclassifierbwd"), x_(x), y_(y), dx_(dx), dy_(dy), loss_(loss)
    {
    }
    void exec(HipProgram &p) override
    {
        const int n = x_->m_dims[0];
        float scale = 1.0f / n;
        if(x_->m_data_type == Tensor::DataType::HALF)
            scale *= p.m_mp_scaling; // loss scaling enters the backward pass here (:1315)
        const SagaTensorView vx = x_->view(), vdx = dx_->view();
        chkSaga(saga_hip_catclassifier_bwd(&vx, &vdx, (const int32_t *)y_->deviceMem(),
                                           (const int32_t *)dy_->deviceMem(),
                                           loss_ ? (float *)loss_->deviceMem() : nullptr, scale, S(p)));
    }
    double bytes() const override { return nbytes(x_) + nbytes(dx_); }
    // the loss scale is a launch argument and changes every step
    bool graphSafe() const override { return x_->m_data_type != Tensor::DataType::HALF; }
    HipOpArgs listInputs() const override { return {{"x", x_}, {"y", y_}, {"dy", dy_}}; }
    HipOpArgs listOutputs() const override
    {
        HipOpArgs r{{"dx", dx_}};
        if(loss_)
            r.push_back({"loss", loss_});
        return r;
    }
    bool killOutput(const std::shared_ptr<HipStorage> &s) override
    {
        if(loss_ && loss_->m_storage == s) {
            loss_.reset();
            return true;
        }
        return false;
    }
};

void catclassifier_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    auto x = p.lower(pu, n.m_inputs["x"]);
    auto y = p.lower(pu, n.m_outputs["y"]);
    pu.fwd(std::make_shared<CatClassifierFwd>(x, y));
    if(p.m_pt == ProgramType::INFERENCE)
        return;
    auto dx = p.lowerGrad(pu, n.m_inputs["x"]);
    auto dy = p.lowerGrad(pu, n.m_outputs["y"]);
    // one loss value per sample; a front end that declares fewer elements gets a batch-sized tensor
    auto lh = n.m_outputs["loss"];
    T loss;
    auto it = p.m_ctx->m_tensors.find(lh);
    if(it != p.m_ctx->m_tensors.end()) {
        loss = it->second;
    } else {
        Dims ld = lh->m_dims.batch(pu.m_batch_size);
        if((int)ld.elements() < (int)x->m_dims[0])
            ld = Dims{(int64_t)(int)x->m_dims[0]};
        loss = std::make_shared<HipTensor>(Tensor::DataType::FLOAT, ld, HipLayout::NCHW, p.m_ctx.get(), lh->m_name);
        p.m_ctx->m_tensors[lh] = loss;
    }
    if(std::max<size_t>(loss->m_dims.elements(), loss->m_storage->m_elements) < (size_t)(int)x->m_dims[0])
        throw std::runtime_error("catclassifier: loss tensor smaller than the batch");
    pu.bwd(std::make_shared<CatClassifierBwd>(x, y, dx, dy, loss));
}
REGISTER_HIP_OP("catclassifier", catclassifier_setup);

// ---------------------------------------------------------------- batch normalisation
// reference: src/cuda/cuda_dnn.cpp:1620-1826 (plain) and :1983-2369 (fused with relu / add)

struct BnInference : public HipOperation {
    const T x_, z_, s_, b_, m_, v_, y_;
    const float eps_;
    const int flags_;
    BnInference(T x, T z, T s, T b, T m, T v, T y, float eps, int flags)
      : HipOperation(flags ? "bninf.fused" : "bninf"), x_(x), z_(z), s_(s), b_(b), m_(m), v_(v), y_(y), eps_(eps), flags_(flags)
    {
    }
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view(), vy = y_->view();
        SagaTensorView vz;
        if(z_)
            vz = z_->view();
        chkSaga(saga_hip_bn_infer(&vx, z_ ? &vz : nullptr, &vy, (const float *)s_->deviceMem(),
                                  (const float *)b_->deviceMem(), (const float *)m_->deviceMem(),
                                  (const float *)v_->deviceMem(), eps_, flags_, S(p)));
    }
    HipOpArgs listInputs() const override
    {
        HipOpArgs r{{"x", x_}, {"s", s_}, {"b", b_}, {"m", m_}, {"v", v_}};
        if(z_)
            r.push_back({"z", z_});
        return r;
    }
    HipOpArgs listOutputs() const override { return {{"y", y_}}; }
    double bytes() const override { return (z_ ? 3 : 2) * nbytes(x_); }
};

struct BnTrain : public HipOperation {
    const T x_, z_, s_, b_, m_, v_, y_, sm_, sv_;
    const float eps_;
    const int flags_;
    float expavg_ = NAN;
    float m_beta_ = 1.0f, v_beta_ = 1.0f; // running statistics are read-modify-write
    std::shared_ptr<ConvStatsLink> stats_; // the producer of x leaves the per-channel sums here
    // fused add + relu on fp16 channels-last tensors: one bit per element (stored y > 0), which the
    // backward pass reads instead of y (the role of cuDNN's reserve space, reference :2095-2136);
    // mask_valid_ says whether the forward pass of this step wrote it
    T mask_;
    bool mask_valid_ = false;
    // a max pooling is the only reader of y and normalises on the fly (BnMaxPoolFwdCodes): this operation then only
    // finalises the statistics and leaves scale and shift in ss_; y stays allocated and unwritten.  applied_ says
    // whether this step's forward pass wrote y after all (the convolution did not deliver its sums).
    T ss_;
    bool applied_ = true;
    BnTrain(HipProgram &p, T x, T z, T s, T b, T m, T v, T y, T sm, T sv, float eps, int flags)
      : HipOperation(flags ? "bntrain.fused" : "bntrain")
      , x_(x), z_(z), s_(s), b_(b), m_(m), v_(v), y_(y), sm_(sm), sv_(sv), eps_(eps), flags_(flags)
    {
        const SagaTensorView vx = x->shapeView();
        p.m_ctx->m_workspace.request(saga_hip_bn_workspace_size(&vx));
    }
    void exec(HipProgram &p) override
    {
        // first step of auto-initialised statistics adopts the batch statistics outright (:1694-1708)
        if(!std::isfinite(expavg_))
            expavg_ = m_->m_auto_initialized ? 1.0f : p.m_pc.bn_expavg;
        const SagaTensorView vx = x_->view(), vy = y_->view();
        SagaTensorView vz;
        if(z_)
            vz = z_->view();
        mask_valid_ = false;
        applied_ = true;
        if(ss_ && stats_ && stats_->valid) {
            const int r = saga_hip_bn_train_fwd_partials(
                &vx, nullptr, nullptr, (const float *)s_->deviceMem(), (const float *)b_->deviceMem(),
                (float *)m_->deviceMem(), (float *)v_->deviceMem(), (float *)sm_->deviceMem(), (float *)sv_->deviceMem(),
                eps_, expavg_, flags_, (const float *)stats_->partial->m_ptr, stats_->rows, nullptr, ss_->deviceMem(),
                ss_->m_dims.elements() * sizeof(float), S(p));
            if(r == 0) {
                stats_->valid = false;
                expavg_ = p.m_pc.bn_expavg;
                applied_ = false;
                return;
            }
            if(r != SAGA_HIP_EUNSUPPORTED)
                chkSaga(r);
        }
        if(stats_ && stats_->valid) {
            stats_->valid = false;
            const int r = saga_hip_bn_train_fwd_partials(
                &vx, z_ ? &vz : nullptr, &vy, (const float *)s_->deviceMem(), (const float *)b_->deviceMem(),
                (float *)m_->deviceMem(), (float *)v_->deviceMem(), (float *)sm_->deviceMem(), (float *)sv_->deviceMem(),
                eps_, expavg_, flags_, (const float *)stats_->partial->m_ptr, stats_->rows,
                mask_ ? (uint8_t *)mask_->deviceMem() : nullptr, p.m_ctx->m_workspace.ptr(), p.m_ctx->m_workspace.size(),
                S(p));
            if(r == 0) {
                expavg_ = p.m_pc.bn_expavg;
                mask_valid_ = mask_ != nullptr;
                return;
            }
            if(r != SAGA_HIP_EUNSUPPORTED)
                chkSaga(r);
        }
        chkSaga(saga_hip_bn_train_fwd(&vx, z_ ? &vz : nullptr, &vy, (const float *)s_->deviceMem(),
                                      (const float *)b_->deviceMem(), (float *)m_->deviceMem(),
                                      (float *)v_->deviceMem(), (float *)sm_->deviceMem(), (float *)sv_->deviceMem(),
                                      eps_, expavg_, flags_, p.m_ctx->m_workspace.ptr(), p.m_ctx->m_workspace.size(),
                                      S(p)));
        expavg_ = p.m_pc.bn_expavg;
    }
    HipOpArgs listInputs() const override
    {
        HipOpArgs r{{"x", x_}, {"s", s_}, {"b", b_}};
        if(z_)
            r.push_back({"z", z_});
        return r;
    }
    HipOpArgs listOutputs() const override
    {
        HipOpArgs r{{"y", y_}, {"m", m_}, {"v", v_}, {"sm", sm_}, {"sv", sv_}};
        if(mask_)
            r.push_back({"mask", mask_});
        if(ss_)
            r.push_back({"ss", ss_});
        return r;
    }
    // statistics pass reads x (unless the producer supplied the sums), normalise pass reads x (+z), writes y
    double bytes() const override
    {
        if(ss_ && stats_) // the partial sums in, a few vectors of C floats out
            return 16.0 * (double)x_->m_dims[1];
        return ((z_ ? 4 : 3) - (stats_ ? 1 : 0) + (mask_ ? 0.0625 : 0)) * nbytes(x_);
    }
    float *getBeta(const T &t) override
    {
        if(t == m_)
            return &m_beta_;
        if(t == v_)
            return &v_beta_;
        return nullptr;
    }
};

struct BnBwd : public HipOperation {
    const std::shared_ptr<BnTrain> fwd_;
    const T dy_, dx_;
    T dz_;
    const T ds_, db_;
    int flags_;
    float dx_beta_ = 0, dz_beta_ = 0, ds_beta_ = 0, db_beta_ = 0;
    std::shared_ptr<BnBwdLinkState> link_; // the last writer of dy leaves it masked, with its per-channel sums
    BnBwd(std::shared_ptr<BnTrain> fwd, T dy, T dx, T dz, T ds, T db, int flags)
      : HipOperation(flags ? "bnbwd.fused" : "bnbwd"), fwd_(fwd), dy_(dy), dx_(dx), dz_(dz), ds_(ds), db_(db), flags_(flags)
    {
    }
    void exec(HipProgram &p) override
    {
        const bool relu = flags_ & SAGA_BN_RELU;
        const SagaTensorView vx = fwd_->x_->view(), vy = fwd_->y_->view(), vdy = dy_->view(), vdx = dx_->view();
        SagaTensorView vdz;
        if(dz_)
            vdz = dz_->view();
        if(link_ && link_->valid) {
            link_->valid = false;
            chkSaga(saga_hip_bn_bwd_linked(&vx, &vdy, &vdx, (const float *)fwd_->s_->deviceMem(),
                                           (const float *)fwd_->sm_->deviceMem(), (const float *)fwd_->sv_->deviceMem(),
                                           (float *)ds_->deviceMem(), (float *)db_->deviceMem(), dx_beta_, ds_beta_,
                                           (const float *)link_->partial->m_ptr, link_->rows, p.m_ctx->m_workspace.ptr(),
                                           p.m_ctx->m_workspace.size(), S(p)));
            return;
        }
        // the bias lets the kernels rebuild the relu mask from x when there is no residual
        // (a forward pass that left the normalising to a pooling wrote no y: the mask is then rebuilt from x)
        chkSaga(saga_hip_bn_bwd_ex(&vx, relu && fwd_->applied_ ? &vy : nullptr, &vdy, &vdx, dz_ ? &vdz : nullptr,
                                (const float *)fwd_->s_->deviceMem(), (const float *)fwd_->b_->deviceMem(),
                                (const float *)fwd_->sm_->deviceMem(),
                                (const float *)fwd_->sv_->deviceMem(), (float *)ds_->deviceMem(),
                                (float *)db_->deviceMem(), dx_beta_, dz_beta_, ds_beta_, flags_,
                                fwd_->mask_valid_ ? (const uint8_t *)fwd_->mask_->deviceMem() : nullptr,
                                p.m_ctx->m_workspace.ptr(), p.m_ctx->m_workspace.size(), S(p)));
    }
    HipOpArgs listInputs() const override
    {
        HipOpArgs r{{"x", fwd_->x_}, {"dy", dy_}, {"s", fwd_->s_}, {"sm", fwd_->sm_}, {"sv", fwd_->sv_}};
        if(flags_ & SAGA_BN_RELU)
            r.push_back({"y", fwd_->y_});
        if(fwd_->mask_)
            r.push_back({"mask", fwd_->mask_});
        return r;
    }
    HipOpArgs listOutputs() const override
    {
        HipOpArgs r{{"dx", dx_}, {"ds", ds_}, {"db", db_}};
        if(dz_)
            r.push_back({"dz", dz_});
        return r;
    }
    bool killOutput(const std::shared_ptr<HipStorage> &s) override
    {
        if(dz_ && dz_->m_storage == s) {
            dz_.reset();
            return true;
        }
        return false;
    }
    // both passes read x and dy (and y when the relu is fused); the second writes dx (and dz)
    double bytes() const override
    {
        const double e = nbytes(dx_);
        if(link_ && !link_->refused) // one pass: x and the masked gradient in, dx out
            return e * (3 + (dx_beta_ != 0 ? 1 : 0));
        const bool reads_y = (flags_ & SAGA_BN_RELU) && (flags_ & SAGA_BN_ADD);
        if(reads_y && dz_ && dz_beta_ == 0) // pass 1: x, y (or its 1-bit mask), dy -> dz ; pass 2: x, dz -> dx
            return e * ((fwd_->mask_ ? 6.0625 : 7) + (dx_beta_ != 0 ? 1 : 0));
        return e * (4 + (reads_y ? 2 : 0) + 1 + (dz_ ? 1 : 0) + (dx_beta_ != 0 ? 1 : 0) +
                    (dz_ && dz_beta_ != 0 ? 1 : 0));
    }
    float *getBeta(const T &t) override
    {
        if(t == dx_)
            return &dx_beta_;
        if(dz_ && t == dz_)
            return &dz_beta_;
        if(t == ds_)
            return &ds_beta_;
        if(t == db_)
            return &db_beta_;
        return nullptr;
    }
};

} // namespace

// Gradients that fan in are summed by letting every writer after the first accumulate.  A 1x1 backward data at
// stride 2 (the projection of a downsampling residual block) reaches one output pixel in four: as the FIRST
// writer it has to fill the other three quarters with zeros, and the dense writer after it then reads all of
// that back to add to it; as the LAST writer it adds to its own quarter and touches nothing else.  Where such
// an operation writes first and other operations write the same tensor later, it is moved behind the last of
// them - nothing in between reads the tensor (it is incomplete until then) or writes what the moved operation
// reads.  Runs before the accumulation factors are assigned.
void reorder_sparse_first_writers(HipOps &ops)
{
    if(getenv("SAGA_HIP_NO_WRITER_REORDER"))
        return;
    for(size_t i = 0; i < ops.size(); i++) {
        auto *conv = dynamic_cast<ConvBwdData *>(ops[i].get());
        if(!conv || conv->cp_.stride < 2 || ((int)conv->w_->m_dims[2] >= conv->cp_.stride && (int)conv->w_->m_dims[3] >= conv->cp_.stride))
            continue;
        const T &t = conv->dx_;
        bool first = true;
        for(size_t k = 0; k < i && first; k++)
            for(const auto &o : ops[k]->listOutputs())
                if(o.second->m_storage == t->m_storage)
                    first = false;
        if(!first)
            continue;
        ssize_t last = -1;
        bool ok = true;
        for(size_t k = i + 1; k < ops.size() && ok; k++) {
            bool writes = false;
            for(const auto &o : ops[k]->listOutputs())
                if(o.second->m_storage == t->m_storage) {
                    // every later writer must be able to go first or to accumulate, on this very tensor
                    if(o.second != t || !ops[k]->getBeta(o.second))
                        ok = false;
                    writes = true;
                }
            if(writes)
                last = (ssize_t)k;
        }
        if(!ok || last < 0)
            continue;
        for(size_t k = i + 1; k <= (size_t)last && ok; k++) {
            for(const auto &in : ops[k]->listInputs())
                if(in.second->m_storage == t->m_storage)
                    ok = false; // somebody reads the sum before it is complete: leave the order alone
            for(const auto &o : ops[k]->listOutputs())
                for(const auto &in : conv->listInputs())
                    if(o.second->m_storage == in.second->m_storage)
                        ok = false;
        }
        if(!ok)
            continue;
        auto moved = ops[i];
        ops.erase(ops.begin() + i);
        ops.insert(ops.begin() + last, moved); // `last` shifted down by one: this is right behind it
        i--;                                     // what slid into position i is looked at next
    }
}

// Training programs: where the gradient of a batch norm's (+ relu) output is written last by a convolution's
// backward data and read by nobody but the norm's backward, that convolution masks the gradient and sums it
// per channel on the way out, and the norm's backward starts from those sums.
void link_bn_backward(HipProgram &p, HipOps &ops)
{
    if(getenv("SAGA_HIP_NO_BNBWD_LINK"))
        return;
    for(size_t ib = 0; ib < ops.size(); ib++) {
        auto *bn = dynamic_cast<BnBwd *>(ops[ib].get());
        if(!bn || bn->link_ || (bn->flags_ & SAGA_BN_ADD) || bn->dz_)
            continue;
        const T &g = bn->dy_, &x = bn->fwd_->x_;
        if(g->m_data_type != Tensor::DataType::HALF || x->m_data_type != Tensor::DataType::HALF ||
           x->m_storage == g->m_storage || x->m_dims.i64() != g->m_dims.i64())
            continue;
        const auto &ex = p.m_ctx->m_exported;
        if(std::any_of(ex.begin(), ex.end(), [&](const auto &e) { return e == g->m_storage; }))
            continue; // the host may look at the unmasked gradient
        ssize_t last_writer = -1;
        bool clean = true;
        for(size_t i = 0; i < ops.size() && clean; i++) {
            if(i == ib)
                continue;
            for(const auto &o : ops[i]->listOutputs())
                if(o.second->m_storage == g->m_storage) {
                    if(i > ib || o.second != g)
                        clean = false;
                    last_writer = (ssize_t)i;
                }
            for(const auto &in : ops[i]->listInputs())
                if(in.second->m_storage == g->m_storage)
                    clean = false;
        }
        if(!clean || last_writer < 0)
            continue;
        auto *conv = dynamic_cast<ConvBwdData *>(ops[last_writer].get());
        if(!conv || conv->dx_ != g)
            continue;
        bn->link_ = conv->linkBnBwd(x, bn->fwd_->s_, bn->fwd_->b_, bn->fwd_->sm_, bn->fwd_->sv_, bn->flags_ & SAGA_BN_RELU);
        if(bn->link_)
            bn->m_kind = "bnbwd.linked";
    }
}

namespace {

bool single_consumer(const Nodes &nodes, const std::shared_ptr<Tensor> &t);

// x0 = normalised input, x1 = residual (optional); flags from the "relu" attribute
void batchnorm_lower(HipProgram &p, HipProgramUnit &pu, const Node &n, std::shared_ptr<Tensor> xh,
                     std::shared_ptr<Tensor> zh, int flags)
{
    auto x = p.lower(pu, xh);
    auto z = zh ? p.lower(pu, zh) : nullptr;
    auto y = p.lowerLike(pu, n.m_outputs["y"], *x);
    auto s = p.lower(pu, n.m_inputs["s"], 2);
    auto b = p.lower(pu, n.m_inputs["b"], 2);
    auto m = p.lower(pu, n.m_inputs["m"], 2);
    auto v = p.lower(pu, n.m_inputs["v"], 2);
    for(const auto &t : {s, b, m, v})
        if(t->m_data_type != Tensor::DataType::FLOAT || (int)t->m_dims.elements() != (int)x->m_dims[1])
            throw std::runtime_error("batchnorm parameters must be fp32 vectors of C elements");
    const float eps = n.m_attributes.get("epsilon", 1e-5f);

    // the operation that alone writes x, if it is a convolution
    auto conv_producer = [&]() -> ConvFwd * {
        ConvFwd *producer = nullptr;
        int writers = 0;
        for(const auto &op : pu.m_fwd)
            for(const auto &o : op->listOutputs())
                if(o.second->m_storage == x->m_storage) {
                    writers++;
                    producer = o.second == x ? dynamic_cast<ConvFwd *>(op.get()) : nullptr;
                }
        return writers == 1 ? producer : nullptr;
    };
    if(p.m_pt == ProgramType::INFERENCE) {
        // conv -> batch norm with nobody else looking at the convolution's output: one kernel
        ConvFwd *producer = conv_producer();
        const auto &ex = p.m_ctx->m_exported;
        const bool held = std::any_of(ex.begin(), ex.end(), [&](const auto &e) { return e == x->m_storage; });
        if(producer && !held && !p.m_pc.disable_op_fusing && single_consumer(pu.m_transformed, xh) &&
           producer->foldBn(s, b, m, v, z, y, eps, flags))
            return;
        pu.fwd(std::make_shared<BnInference>(x, z, s, b, m, v, y, eps, flags));
        return;
    }
    auto sm = std::make_shared<HipTensor>(Tensor::DataType::FLOAT, *m, m->namePostfix("smean"));
    auto sv = std::make_shared<HipTensor>(Tensor::DataType::FLOAT, *v, v->namePostfix("svar"));
    auto f = std::make_shared<BnTrain>(p, x, z, s, b, m, v, y, sm, sv, eps, flags);
    // if the op that wrote x last is a convolution and nothing else writes x, take the sums from it
    if(ConvFwd *producer = conv_producer())
        f->stats_ = producer->offerStats();
    // residual + relu on fp16 channels-last tensors with whole 8-channel vectors, statistics from
    // the convolution: the forward pass also leaves the relu mask, one bit per element
    if(f->stats_ && z && (flags & SAGA_BN_RELU) && (flags & SAGA_BN_ADD) && x->m_data_type == Tensor::DataType::HALF &&
       x->m_dims.size() == 4 && x->cpacked() && y->cpacked() && (int)x->m_dims[1] % 8 == 0 && !getenv("SAGA_HIP_NO_RELU_MASK")) {
        const Dims md{x->m_dims[0], (int64_t)((int)x->m_dims[1] / 8), x->m_dims[2], x->m_dims[3]};
        f->mask_ = std::make_shared<HipTensor>(Tensor::DataType::U8, md, HipLayout::NHWC, p.m_ctx.get(),
                                               n.m_outputs["y"]->namePostfix("relumask"));
    }
    pu.fwd(f);

    auto dx = p.lowerGrad(pu, xh);
    auto dz = zh ? p.lowerGrad(pu, zh) : nullptr;
    auto dy = p.lowerGrad(pu, n.m_outputs["y"]);
    auto ds = p.lowerGrad(pu, n.m_inputs["s"], 2);
    auto db = p.lowerGrad(pu, n.m_inputs["b"], 2);
    pu.bwd(std::make_shared<BnBwd>(f, dy, dx, dz, ds, db, flags));
    p.upd(n.m_inputs["s"], s, ds);
    p.upd(n.m_inputs["b"], b, db);
}

void batchnorm_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    batchnorm_lower(p, pu, n, n.m_inputs["x"], nullptr, 0);
}
REGISTER_HIP_OP("batchnorm", batchnorm_setup);

void batchnorm_fused_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    int flags = 0;
    std::shared_ptr<Tensor> z;
    if(n.m_attributes.get("relu", false))
        flags |= SAGA_BN_RELU;
    if(n.m_inputs.has("x1")) {
        z = n.m_inputs["x1"];
        flags |= SAGA_BN_ADD;
    }
    batchnorm_lower(p, pu, n, n.m_inputs["x0"], z, flags);
}
REGISTER_HIP_OP("batchnorm.persistent", batchnorm_fused_setup);

bool single_consumer(const Nodes &nodes, const std::shared_ptr<Tensor> &t)
{
    int uses = 0;
    for(const auto &n : nodes)
        for(const auto &in : n->m_inputs)
            if(in.second == t)
                uses++;
    return uses == 1;
}

std::shared_ptr<Node> fuse_bn(std::shared_ptr<Node> bn, std::shared_ptr<Node> sum, std::shared_ptr<Node> relu)
{
    auto nn = std::make_shared<Node>("batchnorm.persistent", bn->m_name);
    nn->m_inputs["x0"] = bn->m_inputs["x"];
    if(sum) {
        const bool bn_is_x0 = sum->m_inputs["x0"] == bn->m_outputs["y"];
        nn->m_inputs["x1"] = sum->m_inputs[bn_is_x0 ? "x1" : "x0"];
    }
    for(const char *k : {"s", "b", "m", "v"})
        nn->m_inputs[k] = bn->m_inputs[k];
    if(bn->m_attributes.find("epsilon") != bn->m_attributes.end())
        nn->m_attributes["epsilon"] = bn->m_attributes["epsilon"];
    if(relu)
        nn->m_attributes["relu"] = true;
    nn->m_outputs["y"] = relu ? relu->m_outputs["y"] : bn->m_outputs["y"];
    return nn;
}

// bn,relu / bn,sum,relu runs of ADJACENT nodes become one fused node
// (reference: batchnorm_relu_transform, :2326-2369; that one is limited to fp16 channels-last
// training programs, the kernels here take any type and layout and fuse in inference too).
Nodes batchnorm_relu_transform(HipProgram &p, HipProgramUnit &, const Nodes &nodes)
{
    if(p.m_pc.disable_op_fusing)
        return nodes;
    Nodes r;
    const ssize_t count = nodes.size();
    for(ssize_t i = 0; i < count; i++) {
        std::shared_ptr<Node> n = nodes[i];
        if(n->m_type == "batchnorm") {
            const auto bn_y = n->m_outputs["y"];
            if(i + 1 < count && nodes[i + 1]->m_type == "relu" && nodes[i + 1]->m_inputs["x"] == bn_y &&
               single_consumer(nodes, bn_y)) {
                n = fuse_bn(nodes[i], nullptr, nodes[i + 1]);
                i += 1;
            } else if(i + 2 < count && nodes[i + 1]->m_type == "sum" && nodes[i + 2]->m_type == "relu" &&
                      (nodes[i + 1]->m_inputs["x0"] == bn_y || nodes[i + 1]->m_inputs["x1"] == bn_y) &&
                      nodes[i + 1]->m_inputs["x0"] != nodes[i + 1]->m_inputs["x1"] &&
                      nodes[i + 2]->m_inputs["x"] == nodes[i + 1]->m_outputs["y"] && single_consumer(nodes, bn_y) &&
                      single_consumer(nodes, nodes[i + 1]->m_outputs["y"])) {
                n = fuse_bn(nodes[i], nodes[i + 1], nodes[i + 2]);
                i += 2;
            }
        }
        r.push_back(n);
    }
    return r;
}
REGISTER_HIP_TRANSFORM(500, ProgramType::INFERENCE | ProgramType::TRAINING, batchnorm_relu_transform);

// ---------------------------------------------------------------- pooling
// reference: src/cuda/cuda_dnn.cpp:810-926

struct PoolFwd : public HipOperation {
    const T x_, y_;
    const int mode_, size_, pad_, stride_;
    PoolFwd(T x, T y, int mode, int size, int pad, int stride)
      : HipOperation("poolfwd"), x_(x), y_(y), mode_(mode), size_(size), pad_(pad), stride_(stride)
    {
    }
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view(), vy = y_->view();
        chkSaga(saga_hip_pool_fwd(mode_, &vx, &vy, nullptr, size_, pad_, stride_, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", x_}}; }
    HipOpArgs listOutputs() const override { return {{"y", y_}}; }
    std::string info() const override { return mode_ == SAGA_POOL_MAX ? "max" : "avg"; }
    double bytes() const override { return nbytes(x_) + nbytes(y_); }
};

struct PoolBwd : public HipOperation {
    const T x_, y_, dx_, dy_;
    const int mode_, size_, pad_, stride_;
    float beta_ = 0;
    PoolBwd(T x, T y, T dx, T dy, int mode, int size, int pad, int stride)
      : HipOperation("poolbwd"), x_(x), y_(y), dx_(dx), dy_(dy), mode_(mode), size_(size), pad_(pad), stride_(stride)
    {
    }
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view(), vy = y_->view(), vdy = dy_->view(), vdx = dx_->view();
        chkSaga(saga_hip_pool_bwd(mode_, &vx, &vy, &vdy, &vdx, size_, pad_, stride_, beta_, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", x_}, {"y", y_}, {"dy", dy_}}; }
    HipOpArgs listOutputs() const override { return {{"dx", dx_}}; }
    float *getBeta(const T &t) override { return t == dx_ ? &beta_ : nullptr; }
    double bytes() const override
    {
        return nbytes(dx_) + nbytes(dy_) + (mode_ == SAGA_POOL_MAX ? nbytes(x_) + nbytes(y_) : 0);
    }
};

// Max pooling in a training program, channels-last: the forward pass records the position of every
// maximum in a byte tensor of y's shape and the backward pass reads that instead of x and y.
struct MaxPoolFwdCodes : public HipOperation {
    const T x_, y_, codes_;
    const int size_, pad_, stride_;
    MaxPoolFwdCodes(T x, T y, T codes, int size, int pad, int stride)
      : HipOperation("poolfwd"), x_(x), y_(y), codes_(codes), size_(size), pad_(pad), stride_(stride)
    {
    }
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view(), vy = y_->view();
        chkSaga(saga_hip_maxpool_fwd_codes(&vx, &vy, (uint8_t *)codes_->deviceMem(), size_, pad_, stride_, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", x_}}; }
    HipOpArgs listOutputs() const override { return {{"y", y_}, {"codes", codes_}}; }
    std::string info() const override { return "max+codes"; }
    double bytes() const override { return nbytes(x_) + nbytes(y_) + nbytes(codes_); }
};

struct MaxPoolBwdCodes : public HipOperation {
    const T codes_, dy_, dx_;
    const int size_, pad_, stride_;
    float beta_ = 0;
    MaxPoolBwdCodes(T codes, T dy, T dx, int size, int pad, int stride)
      : HipOperation("poolbwd"), codes_(codes), dy_(dy), dx_(dx), size_(size), pad_(pad), stride_(stride)
    {
    }
    void exec(HipProgram &p) override
    {
        const SagaTensorView vdy = dy_->view(), vdx = dx_->view();
        chkSaga(saga_hip_maxpool_bwd_codes((const uint8_t *)codes_->deviceMem(), &vdy, &vdx, size_, pad_, stride_, beta_,
                                           S(p)));
    }
    HipOpArgs listInputs() const override { return {{"codes", codes_}, {"dy", dy_}}; }
    HipOpArgs listOutputs() const override { return {{"dx", dx_}}; }
    float *getBeta(const T &t) override { return t == dx_ ? &beta_ : nullptr; }
    double bytes() const override { return nbytes(dx_) * (beta_ != 0 ? 2 : 1) + nbytes(dy_) + nbytes(codes_); }
};

// Max pooling right behind a batch norm (+ relu) that nobody else reads: the windows are normalised on the fly
// from the norm's input and the normalised tensor - for a ResNet stem the largest activation of the network - is
// neither written nor read.  bn_: the norm's forward operation, which then only finalises its statistics; if in
// some step it had to normalise itself after all (applied_), this is the plain pooling of its output.
struct BnMaxPoolFwdCodes : public HipOperation {
    const std::shared_ptr<BnTrain> bn_;
    const T y_, codes_;
    const int size_, pad_, stride_;
    BnMaxPoolFwdCodes(std::shared_ptr<BnTrain> bn, T y, T codes, int size, int pad, int stride)
      : HipOperation("poolfwd.bn"), bn_(bn), y_(y), codes_(codes), size_(size), pad_(pad), stride_(stride)
    {
    }
    void exec(HipProgram &p) override
    {
        const SagaTensorView vy = y_->view();
        if(bn_->applied_) {
            const SagaTensorView vx = bn_->y_->view();
            chkSaga(saga_hip_maxpool_fwd_codes(&vx, &vy, (uint8_t *)codes_->deviceMem(), size_, pad_, stride_, S(p)));
            return;
        }
        const SagaTensorView vx = bn_->x_->view();
        chkSaga(saga_hip_maxpool_fwd_codes_bn(&vx, &vy, (uint8_t *)codes_->deviceMem(), size_, pad_, stride_,
                                              (const float *)bn_->ss_->deviceMem(), bn_->flags_, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", bn_->y_}, {"bn-x", bn_->x_}, {"ss", bn_->ss_}}; }
    HipOpArgs listOutputs() const override { return {{"y", y_}, {"codes", codes_}}; }
    std::string info() const override { return "max+codes on bn input"; }
    double bytes() const override { return nbytes(bn_->x_) + nbytes(y_) + nbytes(codes_); }
};

// The backward of that pair in one operation: the gradient of the pooled output goes through the position codes
// straight into the two passes of the norm's backward, and the gradient of the norm's output is never stored.
struct BnBwdPooled : public HipOperation {
    const std::shared_ptr<BnTrain> fwd_;
    const T codes_, dp_, dx_, ds_, db_;
    const int flags_, size_, pad_, stride_;
    float dx_beta_ = 0, ds_beta_ = 0, db_beta_ = 0;
    BnBwdPooled(HipProgram &p, std::shared_ptr<BnTrain> fwd, T codes, T dp, T dx, T ds, T db, int flags, int size, int pad,
                int stride)
      : HipOperation("bnbwd.pooled"), fwd_(fwd), codes_(codes), dp_(dp), dx_(dx), ds_(ds), db_(db), flags_(flags)
      , size_(size), pad_(pad), stride_(stride)
    {
        const SagaTensorView vx = fwd->x_->shapeView(), vdp = dp->shapeView();
        p.m_ctx->m_workspace.request(saga_hip_bn_bwd_pooled_workspace_size(&vx, &vdp, size, pad, stride));
    }
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = fwd_->x_->view(), vdp = dp_->view(), vdx = dx_->view();
        chkSaga(saga_hip_bn_bwd_pooled(&vx, &vdp, (const uint8_t *)codes_->deviceMem(), &vdx,
                                       (const float *)fwd_->s_->deviceMem(), (const float *)fwd_->b_->deviceMem(),
                                       (const float *)fwd_->sm_->deviceMem(), (const float *)fwd_->sv_->deviceMem(),
                                       (float *)ds_->deviceMem(), (float *)db_->deviceMem(), dx_beta_, ds_beta_, flags_, size_,
                                       pad_, stride_, p.m_ctx->m_workspace.ptr(), p.m_ctx->m_workspace.size(), S(p)));
    }
    HipOpArgs listInputs() const override
    {
        return {{"x", fwd_->x_}, {"dp", dp_}, {"codes", codes_}, {"s", fwd_->s_}, {"b", fwd_->b_}, {"sm", fwd_->sm_},
                {"sv", fwd_->sv_}};
    }
    HipOpArgs listOutputs() const override { return {{"dx", dx_}, {"ds", ds_}, {"db", db_}}; }
    // both passes read x, the pooled gradient and the codes; the second writes dx
    double bytes() const override
    {
        return nbytes(dx_) * (3 + (dx_beta_ != 0 ? 1 : 0)) + 2 * (nbytes(dp_) + nbytes(codes_));
    }
    float *getBeta(const T &t) override
    {
        if(t == dx_)
            return &dx_beta_;
        if(t == ds_)
            return &ds_beta_;
        if(t == db_)
            return &db_beta_;
        return nullptr;
    }
};

// what saga_hip_maxpool_*_codes accept (anything else takes the x / y based kernels)
static bool maxpool_codes_fit(const HipTensor &x, const HipTensor &y, const HipTensor *dx, const HipTensor *dy, int size,
                              int pad, int stride)
{
    if(getenv("SAGA_HIP_NO_POOL_CODES"))
        return false;
    if(size < 2 || size > 3 || stride < 1 || stride > size || pad >= size)
        return false;
    const int vn = x.m_data_type == Tensor::DataType::HALF ? 8 : x.m_data_type == Tensor::DataType::FLOAT ? 4 : 0;
    if(!vn || x.m_dims.size() != 4 || (int)x.m_dims[1] % vn)
        return false;
    for(const HipTensor *t : {&x, &y, dx, dy}) {
        if(!t || !t->cpacked() || t->m_data_type != x.m_data_type || t->m_dims.elements() >= ((size_t)1 << 31))
            return false;
        for(int i : {0, 2, 3})
            if((int)t->m_dims[i] > 1 && t->m_strides[i] % vn)
                return false;
    }
    return true;
}

void pooling_setup(HipProgram &p, HipProgramUnit &pu, const Node &n, int mode)
{
    auto x = p.lower(pu, n.m_inputs["x"]);
    auto y = p.lowerLike(pu, n.m_outputs["y"], *x);
    const int size = n.m_attributes.get("global", false) ? (int)x->m_dims[2] : n.m_attributes.get("size", 1);
    const int pad = n.m_attributes.get("pad", 0);
    const int stride = n.m_attributes.get("stride", 1);
    if(p.m_pt == ProgramType::INFERENCE) {
        pu.fwd(std::make_shared<PoolFwd>(x, y, mode, size, pad, stride));
        return;
    }
    auto dx = p.lowerGrad(pu, n.m_inputs["x"]);
    auto dy = p.lowerGrad(pu, n.m_outputs["y"]);
    if(mode == SAGA_POOL_MAX && dx && dy && maxpool_codes_fit(*x, *y, dx.get(), dy.get(), size, pad, stride)) {
        // dense N,H,W,C bytes whatever pitch y has
        auto codes = std::make_shared<HipTensor>(Tensor::DataType::U8, y->m_dims, HipLayout::NHWC, p.m_ctx.get(),
                                                 n.m_outputs["y"]->namePostfix("maxpos"));
        pu.fwd(std::make_shared<MaxPoolFwdCodes>(x, y, codes, size, pad, stride));
        pu.bwd(std::make_shared<MaxPoolBwdCodes>(codes, dy, dx, size, pad, stride));
        return;
    }
    pu.fwd(std::make_shared<PoolFwd>(x, y, mode, size, pad, stride));
    pu.bwd(std::make_shared<PoolBwd>(x, y, dx, dy, mode, size, pad, stride));
}
void maxpool_setup(HipProgram &p, HipProgramUnit &pu, const Node &n) { pooling_setup(p, pu, n, SAGA_POOL_MAX); }
void avgpool_setup(HipProgram &p, HipProgramUnit &pu, const Node &n) { pooling_setup(p, pu, n, SAGA_POOL_AVG); }
REGISTER_HIP_OP("maxpool", maxpool_setup);
REGISTER_HIP_OP("avgpool", avgpool_setup);

// ---------------------------------------------------------------- sum / add / softmax
// reference: src/cuda/cuda_dnn.cpp:1830-1964

struct AddOp : public HipOperation {
    const T a_, b_, c_;
    AddOp(T a, T b, T c) : HipOperation("add"), a_(a), b_(b), c_(c) {}
    void exec(HipProgram &p) override
    {
        const SagaTensorView va = a_->view(), vb = b_->view(), vc = c_->view();
        chkSaga(saga_hip_add(&va, &vb, &vc, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"a", a_}, {"b", b_}}; }
    HipOpArgs listOutputs() const override { return {{"c", c_}}; }
    double bytes() const override { return 3 * nbytes(c_); }
};

// dst = src + beta*dst (reference: CudnnTransform, :72-99); also converts between layouts
struct Transform : public HipOperation {
    const T a_, b_;
    float beta_ = 0;
    Transform(T a, T b, const char *name = "transform") : HipOperation(name), a_(a), b_(b) {}
    void exec(HipProgram &p) override
    {
        const SagaTensorView va = a_->view(), vb = b_->view();
        chkSaga(saga_hip_axpby(&va, &vb, 1.0f, beta_, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"a", a_}}; }
    HipOpArgs listOutputs() const override { return {{"b", b_}}; }
    float *getBeta(const T &t) override { return t == b_ ? &beta_ : nullptr; }
    double bytes() const override { return (beta_ != 0 ? 3 : 2) * nbytes(b_); }
};

// y = x0 + x1 (+ x2 ...).  The reference reads x0 and x1 only (cuda_dnn.cpp:1883-1890) although
// its ONNX loader attaches every input of an n-ary Sum (onnx.cpp:540-553); here all of them are added.
void sum_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    const auto xh = n.m_inputs.getv("x");
    if(xh.empty())
        throw std::runtime_error("sum without inputs");
    std::vector<T> xs;
    for(const auto &h : xh)
        xs.push_back(p.lower(pu, h));
    auto y = p.lowerLike(pu, n.m_outputs["y"], *xs[0]);
    if(xs.size() == 1)
        pu.fwd(std::make_shared<Transform>(xs[0], y));
    else
        pu.fwd(std::make_shared<AddOp>(xs[0], xs[1], y));
    // further writers of y: the program gives every writer after the first beta = 1 (y += x)
    for(size_t i = 2; i < xs.size(); i++)
        pu.fwd(std::make_shared<Transform>(xs[i], y));
    if(p.m_pt == ProgramType::INFERENCE)
        return;
    auto dy = p.lowerGrad(pu, n.m_outputs["y"]);
    for(const auto &h : xh)
        pu.bwd(std::make_shared<Transform>(dy, p.lowerGrad(pu, h)));
}
REGISTER_HIP_OP("sum", sum_setup);

// y = x + b with b either of x's shape or one value per channel (ONNX Add of a bias); inference only
struct AddBias : public HipOperation {
    const T x_, b_, y_;
    AddBias(T x, T b, T y) : HipOperation("add.bias"), x_(x), b_(b), y_(y) {}
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view(), vy = y_->view(), vb = b_->view();
        chkSaga(saga_hip_axpby(&vx, &vy, 1.0f, 0.0f, S(p)));
        chkSaga(saga_hip_bias_add(&vy, &vb, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", x_}, {"b", b_}}; }
    HipOpArgs listOutputs() const override { return {{"y", y_}}; }
};

void add_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    if(p.m_pt != ProgramType::INFERENCE)
        throw std::runtime_error{"Add not supported for backprop"};
    auto x = p.lower(pu, n.m_inputs["x"]);
    auto y = p.lowerLike(pu, n.m_outputs["y"], *x);
    auto bh = n.m_inputs["b"];
    if(bh->m_dims.elements() == x->m_dims.elements()) {
        auto b = p.lower(pu, bh);
        pu.fwd(std::make_shared<AddOp>(x, b, y));
    } else {
        auto b = p.lower(pu, bh);
        if((int)b->m_dims.elements() != (int)x->m_dims[1])
            throw std::runtime_error("add: b must match x or hold one value per channel");
        pu.fwd(std::make_shared<AddBias>(x, b, y));
    }
}
REGISTER_HIP_OP("add", add_setup);

struct Softmax : public HipOperation {
    const T x_, y_;
    Softmax(T x, T y) : HipOperation("softmaxfwd"), x_(x), y_(y) {}
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view(), vy = y_->view();
        chkSaga(saga_hip_softmax(&vx, &vy, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", x_}}; }
    HipOpArgs listOutputs() const override { return {{"y", y_}}; }
};

void softmax_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    if(p.m_pt != ProgramType::INFERENCE)
        throw std::runtime_error{"not supported for training"};
    auto x = p.lower(pu, n.m_inputs["x"]);
    auto y = p.lowerLike(pu, n.m_outputs["y"], *x);
    pu.fwd(std::make_shared<Softmax>(x, y));
}
REGISTER_HIP_OP("softmax", softmax_setup);

// ---------------------------------------------------------------- spatial transform
// Affine grid + bilinear sampler, forward only (reference: CudnnSpatialTransformFwd and
// spatialtransform_setup, :2372-2460).  The kernel samples fp16 and fp32 tensors directly, so the
// convert -> transform -> convert sandwich the reference builds for non-float inputs (:2462-2500)
// is not needed: the arithmetic (fp32 mix of exactly converted inputs, rounded once) is the same.

struct SpatialTransform : public HipOperation {
    const T x_, theta_, y_;
    SpatialTransform(T x, T theta, T y) : HipOperation("spatialtransform"), x_(x), theta_(theta), y_(y) {}
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view(), vy = y_->view();
        chkSaga(saga_hip_spatial_transform(&vx, (const float *)theta_->deviceMem(), &vy, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", x_}, {"theta", theta_}}; }
    HipOpArgs listOutputs() const override { return {{"y", y_}}; }
    double bytes() const override { return nbytes(x_) + nbytes(y_); }
};

void spatialtransform_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    auto x = p.lower(pu, n.m_inputs["x"]);
    auto y = p.lower(pu, n.m_outputs["y"]);
    // during inference the transform is a plain resize unless the node asks otherwise
    const bool disable = p.m_pt == ProgramType::INFERENCE && !n.m_attributes.get("inference", false);
    if(disable && x->m_dims == y->m_dims) {
        pu.fwd(std::make_shared<Transform>(x, y));
        return;
    }
    auto th = n.m_inputs.has("theta") ? n.m_inputs["theta"] : nullptr;
    if(disable || !th) {
        th = makeCPUTensor(Tensor::DataType::FLOAT, Dims{(int64_t)pu.m_batch_size, (int64_t)2, (int64_t)3},
                           "theta.identity");
        auto ta = th->access();
        for(int i = 0; i < pu.m_batch_size; i++) {
            ta->set({i, 0, 0}, 1);
            ta->set({i, 1, 1}, 1);
        }
    }
    auto theta = p.lower(pu, th);
    if(theta->m_data_type != Tensor::DataType::FLOAT || theta->m_dims.elements() != (size_t)(int)x->m_dims[0] * 6 ||
       !theta->rowMajor())
        throw std::runtime_error("spatialtransform: theta must be an fp32 [N,2,3] tensor in row-major order (got " +
                                 theta->info() + " for x " + x->info() + ")");
    if(x->m_data_type != y->m_data_type ||
       (x->m_data_type != Tensor::DataType::FLOAT && x->m_data_type != Tensor::DataType::HALF))
        throw std::runtime_error("spatialtransform: x and y must both be fp32 or both fp16");
    pu.fwd(std::make_shared<SpatialTransform>(x, theta, y));
}
REGISTER_HIP_OP("spatialtransform", spatialtransform_setup);

// ---------------------------------------------------------------- L2 loss, tensor statistics
// loss (reference: CudaLossFwd / CudaLossBwd, src/cuda/cuda_dnn.cpp:1358-1482): forward copies x to y (in
// y's type), backward leaves dx = (x - target) * strength / N (times the loss scale) and the per-sample
// {min, max, mean, mean square} of the residual in mmss.
// stats (reference: CudaStats, :2638-2680): statistics of an already lowered tensor, run in the tail.

struct LossBwd : public HipOperation {
    const T x_, target_, dx_, mmss_;
    const float strength_;
    LossBwd(T x, T target, T dx, T mmss, float strength)
      : HipOperation("lossbwd"), x_(x), target_(target), dx_(dx), mmss_(mmss), strength_(strength)
    {
    }
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view(), vt = target_->view(), vdx = dx_->view();
        const float scale = strength_ / (float)x_->m_dims[0] * p.m_mp_scaling; // :1412, :1419
        chkSaga(saga_hip_loss_bwd(&vx, &vt, &vdx, (float *)mmss_->deviceMem(), scale, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", x_}, {"target", target_}}; }
    HipOpArgs listOutputs() const override { return {{"dx", dx_}, {"mmss", mmss_}}; }
    bool graphSafe() const override { return false; } // the loss scale is a launch argument
};

void loss_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    auto x = p.lower(pu, n.m_inputs["x"]);
    auto y = p.lowerLike(pu, n.m_outputs["y"], *x);
    pu.fwd(std::make_shared<Convert>(x, y, 1.0f));
    if(p.m_pt == ProgramType::INFERENCE)
        return;
    auto dx = p.lowerGrad(pu, n.m_inputs["x"]);
    auto target = p.lowerLike(pu, n.m_inputs["target"], *x);
    auto mmss = p.lower(pu, n.m_outputs["mmss"]);
    if(!dx || !mmss)
        throw std::runtime_error{"loss: needs a gradient for x and the mmss output"};
    pu.bwd(std::make_shared<LossBwd>(x, target, dx, mmss, n.m_attributes.get("strength", 1.0f)));
}
REGISTER_HIP_OP("loss", loss_setup);

struct Stats : public HipOperation {
    const T x_, y_;
    Stats(HipProgram &p, T x, T y) : HipOperation("stats"), x_(x), y_(y)
    {
        p.m_ctx->m_workspace.request(saga_hip_tensor_stats_workspace_size());
    }
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view();
        chkSaga(saga_hip_tensor_stats(&vx, (float *)y_->deviceMem(), p.m_ctx->m_workspace.ptr(), p.m_ctx->m_workspace.size(),
                                      S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", x_}}; }
    HipOpArgs listOutputs() const override { return {{"y", y_}}; }
};

void stats_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    // like the reference, the node inspects a tensor some other node of the program lowered (:2668-2678)
    auto it = p.m_ctx->m_tensors.find(n.m_inputs["x"]);
    if(it == p.m_ctx->m_tensors.end())
        throw std::runtime_error{"x-tensor not found"};
    auto y = p.lower(pu, n.m_outputs["y"]);
    pu.tail(std::make_shared<Stats>(p, it->second, y));
}
REGISTER_HIP_OP("stats", stats_setup);

// ---------------------------------------------------------------- dropout
// Inference: identity (the reference aliases it away, :1576-1616).  Training (:1486-1574): the mask is a
// function of (seed, call number, element index); the forward operation counts its calls and the backward
// operation asks it for the number of the call it answers, so the pair agrees without a stored mask.

struct DropoutFwd : public HipOperation {
    const T x_, y_;
    const float prob_;
    const uint64_t seed_;
    uint64_t calls_ = 0;
    DropoutFwd(T x, T y, float prob, uint64_t seed) : HipOperation("dropoutfwd"), x_(x), y_(y), prob_(prob), seed_(seed) {}
    void exec(HipProgram &p) override
    {
        const SagaTensorView vx = x_->view(), vy = y_->view();
        chkSaga(saga_hip_dropout_fwd(&vx, &vy, prob_, seed_, ++calls_, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"x", x_}}; }
    HipOpArgs listOutputs() const override { return {{"y", y_}}; }
    bool graphSafe() const override { return false; } // the call number is a launch argument
    double bytes() const override { return nbytes(x_) + nbytes(y_); }
};

struct DropoutBwd : public HipOperation {
    const std::shared_ptr<DropoutFwd> fwd_;
    const T dy_, dx_;
    float beta_ = 0;
    DropoutBwd(std::shared_ptr<DropoutFwd> fwd, T dy, T dx) : HipOperation("dropoutbwd"), fwd_(fwd), dy_(dy), dx_(dx) {}
    void exec(HipProgram &p) override
    {
        const SagaTensorView vdy = dy_->view(), vdx = dx_->view();
        chkSaga(saga_hip_dropout_bwd(&vdy, &vdx, fwd_->prob_, fwd_->seed_, fwd_->calls_, beta_, S(p)));
    }
    HipOpArgs listInputs() const override { return {{"dy", dy_}}; }
    HipOpArgs listOutputs() const override { return {{"dx", dx_}}; }
    float *getBeta(const T &t) override { return t == dx_ ? &beta_ : nullptr; }
    bool graphSafe() const override { return false; }
    double bytes() const override { return nbytes(dy_) + nbytes(dx_) * (beta_ != 0 ? 2 : 1); }
};

void dropout_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    auto x = p.lower(pu, n.m_inputs["x"]);
    if(p.m_pt == ProgramType::INFERENCE) {
        p.m_ctx->m_tensors[n.m_outputs["y"]] =
            alias_of(x, x->m_dims, x->m_strides, x->m_offset, n.m_outputs["y"]->namePostfix("nop-dropout"));
        return;
    }
    auto y = p.lowerLike(pu, n.m_outputs["y"], *x);
    const float prob = n.m_attributes.get("prob", 0.5f);
    if(!(prob >= 0.0f && prob < 1.0f))
        throw std::runtime_error{fmt("dropout: prob %f is outside [0, 1)", prob)};
    // a different stream of masks per dropout node of the program
    static const uint64_t base = 0x5a6a5eedull;
    auto fwd = std::make_shared<DropoutFwd>(x, y, prob, base + 0x100000001b3ull * (uint64_t)(pu.m_fwd.size() + 1));
    pu.fwd(fwd);
    if(auto dx = p.lowerGrad(pu, n.m_inputs["x"]))
        pu.bwd(std::make_shared<DropoutBwd>(fwd, p.lowerGrad(pu, n.m_outputs["y"]), dx));
}
REGISTER_HIP_OP("dropout", dropout_setup);

// ---------------------------------------------------------------- reshape / window / concat
// No arithmetic: outputs alias their inputs (reference: :2504-2634).

// A reshape keeps the LOGICAL (N,C,H,W) element order.  Row-major tensors are re-viewed in
// place; a channels-last tensor with H*W > 1 is first copied into row-major order, so that
// both layouts feed the same values to a following fc (the reference aliases the physical
// order instead, which makes its two layouts disagree for such networks).
void reshape_setup(HipProgram &p, HipProgramUnit &pu, const Node &n)
{
    auto xh = n.m_inputs["x"], yh = n.m_outputs["y"];
    auto x = p.lower(pu, xh);
    const Dims ydims = yh->m_dims.batch(pu.m_batch_size);
    const bool training = p.m_pt == ProgramType::TRAINING;
    T flat = x;
    if(!x->rowMajor()) {
        flat = std::make_shared<HipTensor>(x->m_data_type, x->m_dims, HipLayout::NCHW, p.m_ctx.get(),
                                           xh->namePostfix("rowmajor"));
        pu.fwd(std::make_shared<Transform>(x, flat, "reshape.copy"));
    }
    p.m_ctx->m_tensors[yh] =
        alias_of(flat, ydims, hip_strides(ydims, HipLayout::NCHW), flat->m_offset, xh->namePostfix("reshape"));
    if(!training)
        return;
    auto dx = p.lowerGrad(pu, xh);
    if(!dx)
        return;
    T dflat = dx;
    if(!dx->rowMajor()) {
        dflat = std::make_shared<HipTensor>(dx->m_data_type, dx->m_dims, HipLayout::NCHW, p.m_ctx.get(),
                                            xh->namePostfix("rowmajor.grad"));
        pu.bwd(std::make_shared<Transform>(dflat, dx, "reshape.copy"));
    }
    p.m_ctx->m_tensors[yh->grad()] =
        alias_of(dflat, ydims, hip_strides(ydims, HipLayout::NCHW), dflat->m_offset, xh->namePostfix("reshape.grad"));
}
REGISTER_HIP_OP("reshape", reshape_setup);

Nodes window_transform(HipProgram &p, HipProgramUnit &pu, const Nodes &nodes)
{
    Nodes r;
    for(const auto &n : nodes) {
        if(n->m_type != "window") {
            r.push_back(n);
            continue;
        }
        auto x = p.lower(pu, n->m_inputs["x"]);
        auto yh = n->m_outputs["y"];
        const std::vector<int> off = n->m_attributes.get("offset", std::vector<int>{});
        int64_t o = x->m_offset;
        for(size_t i = 0; i < off.size() && i < x->m_strides.size(); i++)
            o += (int64_t)off[i] * x->m_strides[i];
        const Dims yd = yh->m_dims.batch(pu.m_batch_size);
        p.m_ctx->m_tensors[yh] = alias_of(x, yd, x->m_strides, o, yh->namePostfix("alias"));
        if(p.m_pt == ProgramType::TRAINING) {
            if(auto dx = p.lowerGrad(pu, n->m_inputs["x"])) {
                int64_t go = dx->m_offset;
                for(size_t i = 0; i < off.size() && i < dx->m_strides.size(); i++)
                    go += (int64_t)off[i] * dx->m_strides[i];
                p.m_ctx->m_tensors[yh->grad()] = alias_of(dx, yd, dx->m_strides, go, yh->namePostfix("alias.grad"));
            }
        }
    }
    return r;
}
REGISTER_HIP_TRANSFORM(100, ProgramType::INFERENCE | ProgramType::TRAINING, window_transform);

// Every input becomes a strided view into the output at its offset along `axis`, so the
// producers write straight into the concatenated tensor.  Walks the nodes back to front so
// that nested concats resolve outermost first.
Nodes concat_transform(HipProgram &p, HipProgramUnit &pu, const Nodes &nodes)
{
    Nodes r;
    for(ssize_t i = (ssize_t)nodes.size() - 1; i >= 0; i--) {
        const auto &n = nodes[i];
        if(n->m_type != "concat") {
            r.insert(r.begin(), n);
            continue;
        }
        const int axis = n->m_attributes.get("axis", 1);
        auto y = p.lower(pu, n->m_outputs["y"]);
        T dy = p.m_pt == ProgramType::TRAINING ? p.lowerGrad(pu, n->m_outputs["y"]) : nullptr;
        int64_t along = 0;
        for(const auto &xh : n->m_inputs.getv("x")) {
            const Dims xd = xh->m_dims.batch(pu.m_batch_size);
            auto x = alias_of(y, xd, y->m_strides, y->m_offset + along * y->m_strides[axis], xh->namePostfix("alias"));
            x->copyFromHost(*xh); // inputs that carry values (graph inputs) are placed right away
            p.m_ctx->m_tensors[xh] = x;
            if(dy)
                p.m_ctx->m_tensors[xh->grad()] = alias_of(dy, xd, dy->m_strides,
                                                          dy->m_offset + along * dy->m_strides[axis],
                                                          xh->namePostfix("alias.grad"));
            along += (int)xh->m_dims[axis];
        }
    }
    return r;
}
REGISTER_HIP_TRANSFORM(100, ProgramType::INFERENCE | ProgramType::TRAINING, concat_transform);

}  // namespace

// Training programs: a max pooling (with position codes) whose input is the output of a batch norm (+ relu) that
// nothing else touches - no other operation of the program reads or writes that storage (a skip connection, a
// concat buffer the norm writes a slice of), not the host, not the anomaly checks - normalises its windows on the
// fly from the norm's input, and the norm's forward only finalises its statistics.  The norm must get its sums
// from the producing convolution, have no residual, and a backward pass that rebuilds the relu mask from x.
// The backward half: the pooling's backward (codes -> gradient of the norm's output) and the norm's backward that
// alone reads that gradient become one operation, if the fused kernels take the geometry.
static void fuse_bn_pooling_backward(HipProgram &p, HipOps &ops, const std::shared_ptr<BnTrain> &bn, const T &codes, int size,
                                     int pad, int stride)
{
    if(getenv("SAGA_HIP_NO_BN_POOL_BWD_FUSE"))
        return;
    ssize_t ipb = -1, ibn = -1;
    for(size_t i = 0; i < ops.size(); i++) {
        if(auto *pb = dynamic_cast<MaxPoolBwdCodes *>(ops[i].get()); pb && pb->codes_ == codes)
            ipb = (ssize_t)i;
        if(auto *bb = dynamic_cast<BnBwd *>(ops[i].get()); bb && bb->fwd_ == bn)
            ibn = (ssize_t)i;
    }
    if(ipb < 0 || ibn < 0 || ipb > ibn)
        return;
    auto *pb = static_cast<MaxPoolBwdCodes *>(ops[ipb].get());
    auto *bb = static_cast<BnBwd *>(ops[ibn].get());
    const T &g = pb->dx_; // gradient of the norm's output
    if(bb->dy_ != g || bb->link_ || bb->dz_ || pb->beta_ != 0.0f)
        return;
    // nobody else reads or writes that gradient, and the host does not hold it
    for(size_t i = 0; i < ops.size(); i++) {
        if((ssize_t)i == ipb || (ssize_t)i == ibn)
            continue;
        for(const auto &o : ops[i]->listOutputs())
            if(o.second->m_storage == g->m_storage)
                return;
        for(const auto &in : ops[i]->listInputs())
            if(in.second->m_storage == g->m_storage)
                return;
    }
    const auto &ex = p.m_ctx->m_exported;
    if(std::any_of(ex.begin(), ex.end(), [&](const auto &e) { return e == g->m_storage; }))
        return;
    const SagaTensorView vx = bn->x_->shapeView(), vdp = pb->dy_->shapeView();
    if(bb->dx_->m_data_type != bn->x_->m_data_type || !bb->dx_->cpacked() || !pb->dy_->cpacked() ||
       saga_hip_bn_bwd_pooled_workspace_size(&vx, &vdp, size, pad, stride) == 0)
        return;
    auto fused = std::make_shared<BnBwdPooled>(p, bn, codes, pb->dy_, bb->dx_, bb->ds_, bb->db_, bb->flags_, size, pad, stride);
    fused->dx_beta_ = bb->dx_beta_;
    fused->ds_beta_ = bb->ds_beta_;
    fused->db_beta_ = bb->db_beta_;
    ops[ibn] = fused;
    ops.erase(ops.begin() + ipb);
}

void fuse_bn_pooling(HipProgram &p, HipOps &ops)
{
    if(p.m_pc.disable_op_fusing || p.m_pc.anomaly_detect || getenv("SAGA_HIP_NO_BN_POOL_FUSE") ||
       getenv("SAGA_HIP_BN_MASK_FROM_Y"))
        return;
    for(size_t ip = 0; ip < ops.size(); ip++) {
        auto pool = std::dynamic_pointer_cast<MaxPoolFwdCodes>(ops[ip]);
        if(!pool)
            continue;
        const T &x = pool->x_;
        std::shared_ptr<BnTrain> bn;
        bool clean = true;
        for(size_t i = 0; i < ops.size() && clean; i++) {
            if(i == ip)
                continue;
            for(const auto &o : ops[i]->listOutputs())
                if(o.second->m_storage == x->m_storage) {
                    auto f = std::dynamic_pointer_cast<BnTrain>(ops[i]);
                    if(bn || !f || f->y_ != x || i > ip)
                        clean = false;
                    bn = f;
                }
        }
        if(!clean || !bn || !bn->stats_ || bn->z_ || bn->mask_ || bn->ss_ || (bn->flags_ & ~SAGA_BN_RELU))
            continue;
        for(size_t i = 0; i < ops.size() && clean; i++) {
            if(i == ip)
                continue;
            auto *bwd = dynamic_cast<BnBwd *>(ops[i].get());
            if(bwd && bwd->fwd_ == bn) {
                // the norm's own backward lists y but, with the bias at hand and channels-last tensors, does not read it
                if((bn->flags_ & SAGA_BN_RELU) && (!bwd->dx_->cpacked() || !bwd->dy_->cpacked() || !bn->x_->cpacked()))
                    clean = false;
                continue;
            }
            for(const auto &in : ops[i]->listInputs())
                if(in.second->m_storage == x->m_storage)
                    clean = false;
        }
        const auto &ex = p.m_ctx->m_exported;
        if(!clean || std::any_of(ex.begin(), ex.end(), [&](const auto &e) { return e == x->m_storage; }))
            continue;
        // the pooling reads the norm's input in place of its output: same shape, type and channels-last packing
        const HipTensor &bx = *bn->x_;
        if(bx.m_data_type != x->m_data_type || bx.m_dims.i64() != x->m_dims.i64() || !bx.cpacked() ||
           !maxpool_codes_fit(bx, bx, &bx, &bx, pool->size_, pool->pad_, pool->stride_))
            continue;
        const Dims sd{(int64_t)2 * (int64_t)x->m_dims[1]};
        bn->ss_ = std::make_shared<HipTensor>(Tensor::DataType::FLOAT, sd, HipLayout::NCHW, p.m_ctx.get(),
                                              std::string("scaleshift"));
        ops[ip] = std::make_shared<BnMaxPoolFwdCodes>(bn, pool->y_, pool->codes_, pool->size_, pool->pad_, pool->stride_);
        fuse_bn_pooling_backward(p, ops, bn, pool->codes_, pool->size_, pool->pad_, pool->stride_);
    }
}

}  // namespace saga
