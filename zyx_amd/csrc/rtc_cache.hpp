// Run-time compilation of generated HIP source with hiprtc, behind a cache of code objects: in memory for the life
// of the process, and on disk keyed by a hash of the source, the options and the compiler's version -- what zyx's
// C backend does with the shared objects it builds (zyx/src/backend/c.rs:165-186, cache directory
// $XDG_CONFIG_HOME/zyx/cache/c).
#pragma once
#include <memory>
#include <string>
#include <vector>

namespace zk {

// Compiles `source` for gfx950 (or finds the code object in the caches). `options` are hiprtc options; `name` is the
// file name diagnostics carry. Returns null and a message in `err` when the source does not compile.
std::shared_ptr<const std::vector<char>> rtc_compile(const std::string &source, const std::vector<const char *> &options,
                                                     const char *name, std::string &err);

struct RtcCacheStats { uint64_t compiled, memory_hits, disk_hits; };
RtcCacheStats rtc_cache_stats();

} // namespace zk
