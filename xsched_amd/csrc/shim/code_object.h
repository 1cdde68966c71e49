// Kernel argument layouts read from AMDGPU code objects.
//
// To defer a kernel launch the interception shim has to copy the kernel's arguments,
// and hipLaunchKernel() only hands over an array of pointers: the size of every
// argument has to come from somewhere else. The compiler records it in the code
// object: an ELF note (owner "AMDGPU", type 32) holds a MessagePack map whose
// "amdhsa.kernels" entry lists, for every kernel, its arguments with ".offset",
// ".size" and ".value_kind". The reference reads the same note through the comgr
// library (platforms/hip/hal/src/kernel_param.cpp:256-345); this reader needs no
// library: it walks the clang offload bundle, the ELF program headers and the
// MessagePack bytes itself and never reads outside the sizes those headers state.
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

namespace xsched::hip::codeobj
{

struct KernelArg
{
    uint32_t offset = 0; // byte offset in the kernel argument segment
    uint32_t size = 0;   // bytes
};

struct KernelLayout
{
    std::string name;            // ".name": the symbol without the ".kd" suffix
    uint32_t kernarg_bytes = 0;  // ".kernarg_segment_size" (explicit + hidden arguments)
    std::vector<KernelArg> args; // the explicit arguments only, in declaration order
    /// Bytes of a packed buffer that holds every explicit argument at its offset.
    uint32_t ExplicitBytes() const { return args.empty() ? 0 : args.back().offset + args.back().size; }
};

enum class ParseStatus
{
    kOk = 0,
    kNotCodeObject, // neither an offload bundle nor an ELF file
    kCompressed,    // a compressed offload bundle ("CCOB") and no way to unpack it here
    kNoDeviceImage, // a bundle without an amdgcn entry
    kNoMetadata,    // ELF without the AMDGPU metadata note
    kMalformed,     // a header or the MessagePack data points outside the image
};

const char *ToString(ParseStatus status);

/// Reads the layouts of all kernels in `image`: a clang offload bundle, plain or compressed
/// with zstd / zlib (what
/// __hipRegisterFatBinary and hipModuleLoadData receive from hipcc-built programs; the
/// entry whose target names `arch` is taken, else the first amdgcn entry: explicit
/// arguments are laid out alike for every target) or a bare code object (ELF).
/// `bytes` bounds every access; 0 means the caller does not know the size and the sizes
/// in the bundle / ELF headers are trusted.
ParseStatus ReadKernelLayouts(const void *image, size_t bytes, const char *arch,
                              std::vector<KernelLayout> *out);

} // namespace xsched::hip::codeobj
