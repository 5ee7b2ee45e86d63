// ZfpCompressor (custom/compressor/zfpc.h:8-26, zfpc.cpp:23-97): zfp fixed-rate codec
// (default 8 bits per value) on fp32 data as a 2-D field nx = sizes[2], ny = sizes[0]*sizes[1];
// the stream travels in an fp16-typed tensor of (bufsize + 1) / 2 elements.  No zfp library is
// linked: the codec is libplanmoe_hip's, bit-compatible with zfp 0.5.5.
#ifndef PLANMOE_ZFP_COMPRESSOR
#define PLANMOE_ZFP_COMPRESSOR
#include "abstract.h"
#include <hip/hip_runtime_api.h>

class ZfpCompressor : public AbstractCompressor {
public:
    torch::Tensor compress(const torch::Tensor &) override;
    torch::Tensor decompress(const torch::Tensor &) override;
    void          all_to_all(const torch::Tensor &, const torch::Tensor &) override;
    void          set_cuda_stream(const hipStream_t &);
    void          set_compress_rate(const double &);
    ZfpCompressor(std::shared_ptr<AbstractComm>, double = 8.0) noexcept;
    ~ZfpCompressor();

public:
    double            compress_rate;
    void             *buffer;
    size_t            last_bufsize;
    std::vector<long> sizes;
    size_t            length;
    hipStream_t       cuda_stream = nullptr;
};
#endif
