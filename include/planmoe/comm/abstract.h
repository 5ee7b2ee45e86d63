// AbstractComm -- the communication plug-in interface of the reference
// (custom/comm/abstract.h:10-24), kept as the handle type the compressors hold.
// One GPU: IdentityComm copies `length` bytes from input to output on the current stream
// (what NaiveComm::all_to_all, comm/naive.cpp:11-27, does when g_world_size == 1).
#ifndef PLANMOE_ABSTRACT_COMM
#define PLANMOE_ABSTRACT_COMM

#include <ATen/hip/HIPContext.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>
#include <vector>

// what at::cuda::CUDAStream becomes in a hipified torch extension
using PlanMoEStream = c10::hip::HIPStreamMasqueradingAsCUDA;
// RCCL's communicator handle, opaque here (no collective is issued on one GPU)
#ifndef NCCL_H_
typedef struct ncclComm *ncclComm_t;
#endif

class AbstractComm {
public:
    virtual void all_to_all(const torch::Tensor &, const torch::Tensor &, size_t) = 0;
    AbstractComm(std::vector<PlanMoEStream> *, std::vector<ncclComm_t>, const int &, const int &, const int &, const int &);
    virtual void pre_comm(const torch::Tensor &);
    virtual ~AbstractComm();

    std::vector<PlanMoEStream> *stream;
    std::vector<ncclComm_t>     g_nccl_comm;
    int                         g_world_size;
    int                         g_world_rank;
    int                         g_local_size;
    int                         g_local_rank;
};

class IdentityComm : public AbstractComm {
public:
    IdentityComm(std::vector<PlanMoEStream> *, std::vector<ncclComm_t>, const int &, const int &, const int &, const int &);
    void all_to_all(const torch::Tensor &, const torch::Tensor &, size_t) override;
};

#endif // PLANMOE_ABSTRACT_COMM
