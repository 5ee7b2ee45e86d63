// Plug-in point for compressors written against compressor/abstract.h.  The reference picks its
// compressor by name inside get_compressor (custom/custom_kernel.cpp:194-207), so a third-party
// class has to be added to that function's source; here it registers a factory under a name and
// compress_operation(input, name, comm_name) finds it (a registered name takes precedence over
// the built-in "int8", "zfp", "lz" and the default NoCompressor).
#ifndef PLANMOE_COMPRESSOR_REGISTRY
#define PLANMOE_COMPRESSOR_REGISTRY

#include "abstract.h"
#include <string>
#include <vector>

namespace planmoe {

using CompressorFactory = AbstractCompressor *(*)(std::shared_ptr<AbstractComm>);

// defined in the schemoe_custom_kernel extension module; call it from code linked against that module
void register_compressor(const std::string &name, CompressorFactory factory);
std::vector<std::string> registered_compressors();

} // namespace planmoe

#endif // PLANMOE_COMPRESSOR_REGISTRY
