// Int8Compressor (custom/compressor/int8.h:13-28, int8.cpp:7-74): per-row min/max affine
// quantisation to uint8; the codes travel in an fp32-typed tensor of (N + 3) / 4 elements,
// bias and scale stay in the input dtype.
#ifndef PLANMOE_INT8_COMPRESSOR
#define PLANMOE_INT8_COMPRESSOR
#include "abstract.h"

class Int8Compressor : public AbstractCompressor {
public:
    torch::Tensor compress(const torch::Tensor &) override;
    torch::Tensor decompress(const torch::Tensor &) override;
    void          all_to_all(const torch::Tensor &, const torch::Tensor &) override;
    void          pre_comm(const PlanMoEStream *) override;
    Int8Compressor(std::shared_ptr<AbstractComm>);
    ~Int8Compressor() = default;

private:
    torch::Tensor     bias, scale, g_bias, g_scale;
    caffe2::TypeMeta  dtype;
    size_t            length;
    std::vector<long> sizes;
};
#endif
