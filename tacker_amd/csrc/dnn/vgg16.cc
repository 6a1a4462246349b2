#include "vgg16.h"

#include <cmath>
#include <unordered_map>

#include "../Creator.h"
#include "../Logger.h"
#include "../rng.h"

extern Logger logger;
extern std::unordered_map<std::string, void *> fmap;

namespace {

int pad128(int x) { return ((x + 127) / 128) * 128; }

void launch1d(const char *key, long work, void **args, cudaStream_t stream)
{
    long blocks = (work + 255) / 256;
    const long cap = (long)cuCount() * 8;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    TK_SAFE_CALL(tkLaunchKernel(fmap.at(key), dim3((unsigned)blocks).raw(), dim3(256).raw(), args, 0, stream));
}

float *devAlloc(std::vector<void *> &freeList, size_t floats)
{
    float *p = nullptr;
    TK_SAFE_CALL(tkMalloc((void **)&p, floats * sizeof(float)));
    TK_SAFE_CALL(tkMemset(p, 0, floats * sizeof(float)));
    freeList.push_back(p);
    return p;
}

// f16 [rows_pad][cols_pad] with uniform[-1,1]*scale in the top-left rows x cols, zero elsewhere
void *randomHalfMatrix(std::vector<void *> &freeList, tk::Rng &rng, int rows, int cols, int rows_pad,
                       int cols_pad, float scale)
{
    std::vector<uint16_t> host((size_t)rows_pad * cols_pad, 0);
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < cols; ++c)
            host[(size_t)r * cols_pad + c] = tk::float_to_half_bits(rng.uniform(-1.0f, 1.0f) * scale);
    void *p = nullptr;
    TK_SAFE_CALL(tkMalloc(&p, host.size() * 2));
    TK_SAFE_CALL(tkMemcpy(p, host.data(), host.size() * 2, TK_MEMCPY_H2D));
    freeList.push_back(p);
    return p;
}

float *randomBias(std::vector<void *> &freeList, tk::Rng &rng, int n, int n_pad)
{
    std::vector<float> host(n_pad, 0.0f);
    for (int i = 0; i < n; ++i) host[i] = rng.uniform(-0.1f, 0.1f);
    float *p = devAlloc(freeList, n_pad);
    TK_SAFE_CALL(tkMemcpy(p, host.data(), (size_t)n_pad * sizeof(float), TK_MEMCPY_H2D));
    return p;
}

// Shared GEMM machinery of conv and FC layers: persistent objects built once.
class GemmLayer : public LcGemmKernel {
public:
    // tile_end > 0: only the reference tiles [0, tile_end) are computed (the others would be padding)
    GemmLayer(int id, const std::string &name, int M, int N, int K, const void *A, const void *B, float *C,
              int tile_end = 0)
        : M_(M), N_(N), K_(K)
    {
        this->Id = id;
        this->kernelName = name;
        ori_.reset(new OriTZGEMMKernel(id, M, N, K, A, B, C));
        tiles_ = tile_end > 0 ? tile_end : getTZGEMMGridDim(M, N, K)[3];
        gptb_.reset(new GPTBKernel(id, "tzgemm", "gptb_tzgemm", ori_.get(), dim3(cuCount(), 1, 1),
                                   dim3(TZ_THREADS, 1, 1), 0, tiles_));
    }
    std::vector<int> gemmDims() const override { return {M_, N_, K_}; }

protected:
    virtual void before(cudaStream_t stream) = 0;   // operand staging (im2col / pack)
    void executeImpl(cudaStream_t stream) override
    {
        before(stream);
        gptb_->execute(stream);
    }

public:
    void executeMixed(GPTBKernel *be, int be_start, int be_end, cudaStream_t stream,
                      const std::string &variant = "") override
    {
        before(stream);
        if (be_end <= be_start) {
            gptb_->execute(stream);
            return;
        }
        std::unique_ptr<MixKernel> mix(createTzgemmMix(be, gptb_.get(), be_start, be_end, 0, tiles_, variant, 0, 0));
        mix->execute(stream);
    }

protected:
    int M_, N_, K_, tiles_;
    std::unique_ptr<OriTZGEMMKernel> ori_;
    std::unique_ptr<GPTBKernel> gptb_;
};

class ConvKernel : public GemmLayer {
public:
    // act_bias != nullptr: act is the raw output of the previous convolution; its bias and
    // ReLU are applied while the operand is gathered.  pooled: act is that output at twice the
    // height and width, and the 2x2 max pooling between the two layers happens on the way in too.
    ConvKernel(int id, const std::string &name, const float *act, const float *act_bias, bool pooled, int H,
               int W, int C, int c_stride, int Cout, void *A, const void *Wt, float *out)
        : GemmLayer(id, name, pad128(H * W), pad128(Cout), pad128(9 * C), A, Wt, out), act_(act),
          act_bias_(act_bias), pool_(pooled ? 1 : 0), H_(H), W_(W), C_(C), cs_(c_stride), Cout_(Cout), A_(A)
    {
        this->mixable = 2;
        if (pooled && !(C % 8 == 0 && c_stride % 4 == 0))
            logger.ERROR("vgg16: a pooled input needs a channel count that is a multiple of 8");
    }
    // {n,c,h,w, k,c,kh,kw, pad,pad, stride,stride, dil,dil}
    std::vector<int> getArgs() override { return {1, C_, H_, W_, Cout_, C_, 3, 3, 1, 1, 1, 1, 1, 1}; }

protected:
    void before(cudaStream_t stream) override
    {
        int KH = 3, KW = 3, pad = 1, stride = 1, Ho = H_, Wo = W_, Kp = K_;
        int relu = 1;
        if (C_ % 8 == 0 && cs_ % 4 == 0) {   // every layer but the first: each activation read once
            void *args[] = {&act_, &H_, &W_, &C_, &cs_, &A_, &Kp, &act_bias_, &relu, &pool_};
            launch1d("im2col3x3_scatter_nhwc_f16", (long)H_ * W_ * (C_ / 8), args, stream);
            return;
        }
        // the first layer (3 channels): an operand buffer of its own, zeroed once, of which only the
        // columns that hold data are rewritten
        int Kw = (9 * C_ + 7) / 8 * 8;
        void *args[] = {&act_, &H_, &W_, &C_, &cs_, &KH, &KW, &pad, &stride, &Ho, &Wo, &A_, &Kp, &act_bias_, &relu, &Kw};
        launch1d("im2col_nhwc_f16", (long)Ho * Wo * Kw, args, stream);
    }

private:
    const float *act_;
    const float *act_bias_;
    int pool_;
    int H_, W_, C_, cs_, Cout_;
    void *A_;
};

class FcKernel : public GemmLayer {
public:
    // C[128][out_pad] = X[128][K] * W[out_pad][K]^T with the batch-1 activation in row 0 of X, taken
    // from src with stride src_stride.  The activation is the M side so that the reference tiles that
    // hold the result, row 0 .. 63 of C, are the first out_pad / 64 of the tile order: only those are
    // launched, every one of them streams weights nobody else reads, and rows 64 .. 127 of C (all
    // padding) stay as allocated.
    // pool_W > 0: src is the raw output of the last convolution, [.][pool_W][pool_ld] with pool_C
    // channels, and the 2x2 max pooling in front of the classifier happens while the row is packed
    FcKernel(int id, const std::string &name, const float *src, long src_stride, const float *src_bias,
             int src_relu, int in_features, int out_features, const void *Wt, void *X, float *out,
             int pool_W = 0, int pool_ld = 0, int pool_C = 0)
        : GemmLayer(id, name, 128, pad128(out_features), pad128(in_features), X, Wt, out,
                    pad128(out_features) / TZ_REF_TILE),
          src_(src), stride_(src_stride), bias_(src_bias), relu_(src_relu), in_(in_features), out_(out_features),
          X_(X), poolW_(pool_W), poolLd_(pool_ld), poolC_(pool_C)
    {
        this->mixable = 1;
    }
    std::vector<int> getArgs() override { return {M_, N_, K_}; }

protected:
    void before(cudaStream_t stream) override
    {
        if (poolW_ > 0) {
            void *args[] = {&src_, &poolW_, &poolLd_, &poolC_, &bias_, &relu_, &in_, &X_};
            launch1d("pack_fc_input_pooled", in_, args, stream);
            return;
        }
        void *args[] = {&src_, &stride_, &bias_, &relu_, &in_, &X_};
        launch1d("pack_fc_input", in_, args, stream);
    }

private:
    const float *src_;
    long stride_;
    const float *bias_;
    int relu_, in_, out_;
    void *X_;
    int poolW_, poolLd_, poolC_;
};

}  // namespace

struct VGG16::Impl {
    std::vector<void *> freeList;
    std::vector<float> hostInput;
    float *input = nullptr;
    std::vector<VGG16::Act> convOut;   // the 13 convolutions, then the 3 fully connected layers
    float *logits = nullptr;
    long logitsStride = 0;
};

VGG16::VGG16(int taskId, const VGG16Options &o) : Task(taskId, "vgg16"), opt(o), impl(new Impl)
{
    taskType = LC;
    if (opt.height % 32 || opt.width % 32) logger.ERROR("vgg16: input resolution must be a multiple of 32");
    tk::Rng rng(opt.seed);
    auto &fl = impl->freeList;

    int H = opt.height, W = opt.width, C = 3, ld = 3;
    impl->hostInput.resize((size_t)H * W * 3);
    for (auto &v : impl->hostInput) v = rng.uniform();
    impl->input = devAlloc(fl, impl->hostInput.size());
    InputHost[0] = impl->hostInput.data();
    Input[0] = impl->input;
    InputSize[0] = (int)(impl->hostInput.size() * sizeof(float));

    // the largest im2col operand of the network, shared by every conv layer
    size_t maxA = 0;
    {
        int h = H, w = W, c = 3;
        const int plan[] = {64, 64, -1, 128, 128, -1, 256, 256, 256, -1, 512, 512, 512, -1, 512, 512, 512, -1};
        for (int p : plan) {
            if (p < 0) { h /= 2; w /= 2; continue; }
            maxA = std::max(maxA, (size_t)pad128(h * w) * pad128(9 * c));
            c = p;
        }
    }
    void *Abuf = nullptr;
    TK_SAFE_CALL(tkMalloc(&Abuf, maxA * 2));
    TK_SAFE_CALL(tkMemset(Abuf, 0, maxA * 2));
    fl.push_back(Abuf);

    // A convolution leaves 1.1 * A * B^T in its output buffer; bias and ReLU are applied by
    // whatever reads that buffer next (the next layer's operand gather, or the pooling).
    const float *act = impl->input;
    const float *act_bias = nullptr;   // bias the reader of act still has to apply
    int id = 100;
    const int plan[] = {64, 64, -1, 128, 128, -1, 256, 256, 256, -1, 512, 512, 512, -1, 512, 512, 512, -1};
    // A pooling layer is not a kernel either: the next convolution's operand, or the classifier's
    // input row, is built from the 2x2 maxima.
    bool pooled = false;
    int unpooled_W = 0;   // width of the raw convolution output a pending pooling reads
    int block = 1, layer = 1;
    const int n_plan = (int)(sizeof(plan) / sizeof(plan[0]));
    for (int step = 0; step < n_plan; ++step) {
        const int p = plan[step];
        if (p < 0) {
            pooled = true;
            unpooled_W = W;
            H /= 2;
            W /= 2;
            block++;
            layer = 1;
            continue;
        }
        const int Cout = p, Np = pad128(Cout), Kp = pad128(9 * C);
        const std::string name = "conv" + std::to_string(block) + "_" + std::to_string(layer++);
        void *Wt = randomHalfMatrix(fl, rng, Cout, 9 * C, Np, Kp, std::sqrt(2.0f / (9 * C)));
        float *bias = randomBias(fl, rng, Cout, Np);
        float *out = devAlloc(fl, (size_t)pad128(H * W) * Np);
        void *operand = Abuf;
        if (C % 8 != 0) {   // gathered, and only its data columns rewritten: needs zeros nobody else disturbs
            TK_SAFE_CALL(tkMalloc(&operand, (size_t)pad128(H * W) * Kp * 2));
            TK_SAFE_CALL(tkMemset(operand, 0, (size_t)pad128(H * W) * Kp * 2));
            fl.push_back(operand);
        }
        addKernel(new ConvKernel(id++, "Convolution_" + name, act, act_bias, pooled, H, W, C, ld, Cout, operand, Wt,
                                 out));
        pooled = false;
        impl->convOut.push_back(Act{out, H, W, Cout, Np, Wt, bias, Np, Kp});
        act = out;
        act_bias = bias;
        C = Cout;
        ld = Np;
    }
    // classifier: 512*(H/32)*(W/32) -> 4096 -> 4096 -> classes; activations travel as
    // row 0 of the previous FC output, bias+ReLU applied while packing the next input
    const int feat = H * W * C;   // NHWC flatten (ld == C == 512 here)
    void *X1 = nullptr, *X2 = nullptr, *X3 = nullptr;
    auto halfBuf = [&](void **p, size_t n) {
        TK_SAFE_CALL(tkMalloc(p, n * 2));
        TK_SAFE_CALL(tkMemset(*p, 0, n * 2));
        fl.push_back(*p);
    };
    halfBuf(&X1, (size_t)128 * pad128(feat));
    halfBuf(&X2, (size_t)128 * 4096);
    halfBuf(&X3, (size_t)128 * 4096);
    void *W1 = randomHalfMatrix(fl, rng, 4096, feat, 4096, pad128(feat), std::sqrt(2.0f / feat));
    void *W2 = randomHalfMatrix(fl, rng, 4096, 4096, 4096, 4096, std::sqrt(2.0f / 4096));
    void *W3 = randomHalfMatrix(fl, rng, opt.classes, 4096, pad128(opt.classes), 4096, std::sqrt(2.0f / 4096));
    float *b1 = randomBias(fl, rng, 4096, 4096), *b2 = randomBias(fl, rng, 4096, 4096);
    float *o1 = devAlloc(fl, (size_t)128 * 4096), *o2 = devAlloc(fl, (size_t)128 * 4096);
    float *o3 = devAlloc(fl, (size_t)128 * pad128(opt.classes));
    // act is conv5_3's raw output; its pooling, bias and ReLU happen while fc1's input is packed
    addKernel(new FcKernel(id++, "Dot_fc1", act, 1, act_bias, 1, feat, 4096, W1, X1, o1, pooled ? unpooled_W : 0, ld, C));
    addKernel(new FcKernel(id++, "Dot_fc2", o1, 1, b1, 1, 4096, 4096, W2, X2, o2));
    addKernel(new FcKernel(id++, "Dot_fc3", o2, 1, b2, 1, 4096, opt.classes, W3, X3, o3));
    impl->convOut.push_back(Act{o1, 1, 1, 4096, 4096, W1, b1, 4096, pad128(feat)});
    impl->convOut.push_back(Act{o2, 1, 1, 4096, 4096, W2, b2, 4096, 4096});
    impl->convOut.push_back(Act{o3, 1, 1, opt.classes, pad128(opt.classes), W3, nullptr, pad128(opt.classes), 4096});
    impl->logits = o3;
    impl->logitsStride = 1;
}

VGG16::~VGG16()
{
    for (auto *k : kernels) delete k;
    for (void *p : impl->freeList) tkErrCheck(tkFree(p));
}

void VGG16::initExecution()
{
    TK_SAFE_CALL(tkMemcpy(Input[0], InputHost[0], (size_t)InputSize[0], TK_MEMCPY_H2D));
}

const float *VGG16::logits(long *stride) const
{
    if (stride) *stride = impl->logitsStride;
    return impl->logits;
}

VGG16::Act VGG16::activation(int conv_index) const { return impl->convOut.at(conv_index); }

Task *createTask(const std::string &model)
{
    if (model == "vgg16") return new VGG16(1);
    logger.ERROR("createTask: model not found: " + model);
}
