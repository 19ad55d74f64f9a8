// TEST INFRASTRUCTURE ONLY.  Which storage backend holds a block when several are configured:
// the reference computes std::hash<std::string_view> over the 16 id bytes modulo the number of
// backends (ucm/store/detail/type/types.h:39-45, ucm/store/posix/cc/space_layout.cc:164-170).
// The hash is the C++ standard library's, so the checker calls the same routine.
#include <cstddef>
#include <cstdint>
#include <functional>
#include <string_view>

extern "C" uint64_t oracle_block_id_hash(const uint8_t* id)
{
    return (uint64_t)std::hash<std::string_view>{}(std::string_view(reinterpret_cast<const char*>(id), 16));
}
