// AbstractCompressor -- the compressor plug-in interface of the reference
// (custom/compressor/abstract.h:11-22): same virtuals, constructor and public members.
#ifndef PLANMOE_ABSTRACT_COMPRESSOR
#define PLANMOE_ABSTRACT_COMPRESSOR

#include "../comm/abstract.h"
#include <memory>

class AbstractCompressor {
public:
    virtual torch::Tensor compress(const torch::Tensor &)                          = 0;
    virtual torch::Tensor decompress(const torch::Tensor &)                        = 0;
    virtual void          all_to_all(const torch::Tensor &, const torch::Tensor &) = 0;
    virtual void          pre_comm(const PlanMoEStream *);
    AbstractCompressor(std::shared_ptr<AbstractComm>);
    virtual ~AbstractCompressor();

    torch::Tensor                 g_output;
    std::shared_ptr<AbstractComm> comm_ptr;
};

#endif // PLANMOE_ABSTRACT_COMPRESSOR
