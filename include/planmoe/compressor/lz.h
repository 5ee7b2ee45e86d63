// LzCompressor (custom/compressor/lz.h:13-24, lz.cpp:3-73): the GPULZ lossless codec.  compress
// returns its input untouched and keeps the four stream tensors (offset tables, flag bytes,
// token bytes); all_to_all ships those four whole; decompress decodes into the tensor it is
// handed (g_output, a zeroed twin of the input) and returns it.  The codec is libplanmoe_hip's,
// byte-compatible with the reference's streams; the data must be float32 (lz.cpp hands
// data_ptr<float>() to the kernels, gpulz.cu:15,451).
#ifndef PLANMOE_LZ_COMPRESSOR
#define PLANMOE_LZ_COMPRESSOR
#include "abstract.h"

class LzCompressor : public AbstractCompressor {
public:
    torch::Tensor compress(const torch::Tensor &) override;
    torch::Tensor decompress(const torch::Tensor &) override;
    void          all_to_all(const torch::Tensor &, const torch::Tensor &) override;
    LzCompressor(std::shared_ptr<AbstractComm> comm_ptr);

private:
    torch::Tensor flagArrOffsetGlobal, compressedDataOffsetGlobal, flagArrGlobal, compressedDataGlobal;
    torch::Tensor g_flagArrOffsetGlobal, g_compressedDataOffsetGlobal, g_flagArrGlobal, g_compressedDataGlobal;
    torch::Tensor workspace;
};
#endif
