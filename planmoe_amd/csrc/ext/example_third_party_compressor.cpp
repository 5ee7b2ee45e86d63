// A compressor written by a third party against include/planmoe/compressor/abstract.h alone: it
// ships the tensor as fp16 ("half") and widens it again on the receive side.  Built by
// ext/build.py into libexample_third_party_compressor.so, which links against the
// schemoe_custom_kernel module for the base-class symbols; register_example_compressor() puts it
// into the registry under the name "half", after which
// compress_operation(x, "half", "naive") -> comm_operation -> decompress_operation runs it.
#include "planmoe/compressor/abstract.h"
#include "planmoe/compressor/registry.h"

class HalfCompressor : public AbstractCompressor {
public:
    explicit HalfCompressor(std::shared_ptr<AbstractComm> comm_ptr) : AbstractCompressor(comm_ptr) {}
    torch::Tensor compress(const torch::Tensor &input) override
    {
        dtype = input.scalar_type();
        torch::Tensor out = input.to(at::kHalf);
        g_output = at::empty_like(out);
        for (auto &s : *comm_ptr->stream) g_output.record_stream(s);
        return out;
    }
    torch::Tensor decompress(const torch::Tensor &input) override { return input.to(dtype); }
    void all_to_all(const torch::Tensor &input, const torch::Tensor &output) override
    {
        comm_ptr->all_to_all(input, output, input.nbytes());
    }

private:
    at::ScalarType dtype = at::kFloat;
};

extern "C" void register_example_compressor()
{
    planmoe::register_compressor("half", [](std::shared_ptr<AbstractComm> c) -> AbstractCompressor * {
        return new HalfCompressor(c);
    });
}
