// Driver for tests/test_shim_cpu.py: the code-object reader of the interception shim, built
// with the address and undefined-behaviour sanitizers, over damaged copies of real images.
//   code_object_fuzz <rounds> <image file>...
// Every image is read intact (must succeed), then `rounds` times with a few random bytes
// changed, and at every truncation length of a coarse grid, each time from a heap copy of
// exactly the stated size, so that any read past it is caught. Prints one line per image.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iterator>
#include <memory>
#include <vector>

#include "code_object.h"

using namespace xsched::hip::codeobj;

static uint64_t g_state = 0x9E3779B97F4A7C15ull;
static uint64_t Next() { g_state ^= g_state << 13; g_state ^= g_state >> 7; g_state ^= g_state << 17; return g_state; }

static ParseStatus ReadCopy(const std::vector<uint8_t> &image, size_t bytes, size_t *kernels)
{
    std::unique_ptr<uint8_t[]> exact(new uint8_t[bytes ? bytes : 1]);
    memcpy(exact.get(), image.data(), bytes);
    std::vector<KernelLayout> out;
    const ParseStatus status = ReadKernelLayouts(exact.get(), bytes, "gfx950", &out);
    if (kernels) *kernels = out.size();
    return status;
}

int main(int argc, char **argv)
{
    if (argc < 3) return 2;
    const int rounds = atoi(argv[1]);
    for (int f = 2; f < argc; ++f) {
        std::ifstream in(argv[f], std::ios::binary);
        std::vector<uint8_t> file((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
        // the image proper: from the bundle magic (plain or compressed) or the ELF magic on
        size_t at = 0;
        const char *magics[] = { "__CLANG_OFFLOAD_BUNDLE__", "CCOB" };
        const bool host_elf = file.size() > 20 && memcmp(file.data(), "\177ELF", 4) == 0 && file[18] != 224; // e_machine: not AMDGPU
        if (host_elf) {
            for (const char *m : magics) {
                for (size_t i = 0; i + strlen(m) <= file.size(); ++i) {
                    if (memcmp(file.data() + i, m, strlen(m)) == 0) { at = i; goto found; }
                }
            }
        }
    found:
        std::vector<uint8_t> image(file.begin() + at, file.end());
        size_t kernels = 0;
        const ParseStatus intact = ReadCopy(image, image.size(), &kernels);
        if (intact != ParseStatus::kOk || kernels == 0) {
            printf("%s: intact image not read: %s\n", argv[f], ToString(intact));
            return 1;
        }
        size_t ok = 0, refused = 0;
        for (int r = 0; r < rounds; ++r) {
            std::vector<uint8_t> damaged = image;
            const int flips = 1 + (int)(Next() % 8);
            for (int i = 0; i < flips; ++i) damaged[Next() % damaged.size()] = (uint8_t)Next();
            (ReadCopy(damaged, damaged.size(), nullptr) == ParseStatus::kOk ? ok : refused)++;
        }
        for (size_t cut = 1; cut < image.size(); cut += 1 + image.size() / 257) { // a size of 0 means "unknown"
            (ReadCopy(image, cut, nullptr) == ParseStatus::kOk ? ok : refused)++;
        }
        printf("%s: %zu kernels; damaged copies read %zu, refused %zu\n", argv[f], kernels, ok, refused);
    }
    return 0;
}
