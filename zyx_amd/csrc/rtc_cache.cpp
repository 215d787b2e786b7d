#include "rtc_cache.hpp"

#include <hip/hiprtc.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <sys/stat.h>
#include <unistd.h>

namespace zk {

namespace {

std::mutex g_mu;
std::map<std::pair<uint64_t, uint64_t>, std::shared_ptr<const std::vector<char>>> g_mem;
RtcCacheStats g_stats{0, 0, 0};

// two independent 64-bit hashes of the key text: the first names the file, the second is stored inside it, so a
// collision of the name alone cannot hand back another kernel's code
uint64_t fnv1a(const std::string &s, uint64_t h) {
    for (unsigned char ch : s) {
        h ^= ch;
        h *= 0x100000001b3ull;
    }
    return h;
}

struct FileHeader {
    char magic[8]; // "ZHIPRTC1"
    uint64_t check, code_bytes;
};

// Directory of the on-disk cache, or "" when it is switched off (ZYX_HIP_CACHE=0) or no home is known.
// ZYX_HIP_CACHE_DIR overrides; otherwise the reference's rule with its own leaf: $XDG_CONFIG_HOME (absolute) or
// $HOME/.config, then zyx/cache/hip.
std::string cache_dir() {
    if (const char *off = getenv("ZYX_HIP_CACHE"))
        if (off[0] == '0') return "";
    if (const char *d = getenv("ZYX_HIP_CACHE_DIR")) return d;
    std::string base;
    if (const char *x = getenv("XDG_CONFIG_HOME"))
        if (x[0] == '/') base = x;
    if (base.empty())
        if (const char *h = getenv("HOME"))
            if (h[0] == '/') base = std::string(h) + "/.config";
    return base.empty() ? "" : base + "/zyx/cache/hip";
}

void make_dirs(const std::string &path) {
    for (size_t i = 1; i <= path.size(); i++)
        if (i == path.size() || path[i] == '/') (void)mkdir(path.substr(0, i).c_str(), 0755);
}

std::shared_ptr<const std::vector<char>> read_cached(const std::string &file, uint64_t check) {
    FILE *f = fopen(file.c_str(), "rb");
    if (!f) return nullptr;
    FileHeader h{};
    std::shared_ptr<std::vector<char>> code;
    if (fread(&h, sizeof h, 1, f) == 1 && memcmp(h.magic, "ZHIPRTC1", 8) == 0 && h.check == check && h.code_bytes > 0 &&
        h.code_bytes < (1ull << 30)) {
        code = std::make_shared<std::vector<char>>(h.code_bytes);
        if (fread(code->data(), 1, h.code_bytes, f) != h.code_bytes || fgetc(f) != EOF) code.reset(); // truncated or trailing bytes
    }
    fclose(f);
    return code;
}

void write_cached(const std::string &dir, const std::string &file, uint64_t check, const std::vector<char> &code) {
    make_dirs(dir);
    // written under a private name, then renamed: readers see nothing or the whole file
    const std::string tmp = file + ".tmp" + std::to_string((long)getpid());
    FILE *f = fopen(tmp.c_str(), "wb");
    if (!f) return;
    FileHeader h{};
    memcpy(h.magic, "ZHIPRTC1", 8);
    h.check = check;
    h.code_bytes = code.size();
    const bool ok = fwrite(&h, sizeof h, 1, f) == 1 && fwrite(code.data(), 1, code.size(), f) == code.size();
    if (fclose(f) != 0 || !ok || rename(tmp.c_str(), file.c_str()) != 0) (void)unlink(tmp.c_str());
}

} // namespace

RtcCacheStats rtc_cache_stats() {
    std::lock_guard<std::mutex> lk(g_mu);
    return g_stats;
}

std::shared_ptr<const std::vector<char>> rtc_compile(const std::string &source, const std::vector<const char *> &options,
                                                     const char *name, std::string &err) {
    int major = 0, minor = 0;
    (void)hiprtcVersion(&major, &minor);
    std::string key = "hiprtc " + std::to_string(major) + "." + std::to_string(minor) + "\n";
    for (const char *o : options) key += std::string(o) + "\n";
    key += source;
    const uint64_t h1 = fnv1a(key, 0xcbf29ce484222325ull), h2 = fnv1a(key, 0x84222325cbf29ce4ull) ^ (uint64_t)key.size();
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_mem.find({h1, h2});
    if (it != g_mem.end()) {
        g_stats.memory_hits++;
        return it->second;
    }
    const std::string dir = cache_dir();
    char fname[40];
    snprintf(fname, sizeof fname, "/%016llx.hsaco", (unsigned long long)h1);
    const std::string file = dir + fname;
    if (!dir.empty())
        if (auto code = read_cached(file, h2)) {
            g_stats.disk_hits++;
            g_mem[{h1, h2}] = code;
            return code;
        }
    hiprtcProgram prog;
    if (hiprtcCreateProgram(&prog, source.c_str(), name, 0, nullptr, nullptr) != HIPRTC_SUCCESS) {
        err = "hiprtcCreateProgram failed";
        return nullptr;
    }
    const hiprtcResult rc = hiprtcCompileProgram(prog, (int)options.size(), const_cast<const char **>(options.data()));
    if (rc != HIPRTC_SUCCESS) {
        size_t ls = 0;
        hiprtcGetProgramLogSize(prog, &ls);
        std::string log(ls, 0);
        if (ls) hiprtcGetProgramLog(prog, &log[0]);
        err = std::string("hiprtc: ") + hiprtcGetErrorString(rc) + ": " + log.substr(0, 800);
        hiprtcDestroyProgram(&prog);
        return nullptr;
    }
    size_t cs = 0;
    hiprtcGetCodeSize(prog, &cs);
    auto code = std::make_shared<std::vector<char>>(cs);
    hiprtcGetCode(prog, code->data());
    hiprtcDestroyProgram(&prog);
    g_stats.compiled++;
    g_mem[{h1, h2}] = code;
    if (!dir.empty()) write_cached(dir, file, h2, *code);
    return code;
}

} // namespace zk
