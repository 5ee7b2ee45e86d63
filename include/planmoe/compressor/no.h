// NoCompressor (custom/compressor/no.h, no.cpp:3-20)
#ifndef PLANMOE_NO_COMPRESSOR
#define PLANMOE_NO_COMPRESSOR
#include "abstract.h"

class NoCompressor : public AbstractCompressor {
public:
    torch::Tensor compress(const torch::Tensor &) override;
    torch::Tensor decompress(const torch::Tensor &) override;
    void          all_to_all(const torch::Tensor &, const torch::Tensor &) override;
    NoCompressor(std::shared_ptr<AbstractComm> comm_ptr);
};
#endif
