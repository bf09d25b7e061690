// Launch-plan cache of the chunked forward entry point (host code only).
//
// The reference keeps, for flame_sdpa_chunked_bf16, a cache from problem shape to the (query chunk, key
// chunk) pair that its autotuner measured fastest, with counters that its telemetry reads and an
// optional file behind it (reference: cuda/src/flame_sdpa_stub.cu:38-650, :1080-1379; the counters'
// layout cuda/include/flame_cuda_common.cuh:72-98).  The one choice the kernels of this library leave
// open for a problem without mask or bias is the query tile of a workgroup, 128 or 256 rows (the key
// tile is always 64), normally made by a rule on the number of workgroups per compute unit.  This cache
// remembers that choice per shape; on a miss it either takes the rule's answer or, when measuring is on,
// times both tiles on the caller's own problem with HIP events and keeps the faster.
//
// Same environment variables, counters and file format as the reference, so that its telemetry and a
// cache file written by either side stay readable:
//   FLAME_SDPA_AUTOTUNE (default on)      use the cache and measure on a miss; off = the rule, no counters
//   FLAME_SDPA_QCHUNK                     force the query tile (rounded to 128 or 256)
//   FLAME_SDPA_AUTOTUNE_WARMUPS / _REPEATS / _TIE_EPS_PCT   1 / 3 / 2: the measurement
//   FLAME_SDPA_AUTOTUNE_PERSIST, FLAME_SDPA_AUTOTUNE_CACHE, FLAME_SDPA_AUTOTUNE_CACHE_LIMIT, FLAME_SDPA_FLUSH_INSERTS
// File: one JSON object per line, {"meta":{"version":1,...}} first, then
// {"key":{"B":..,"H":..,"Q":..,"K":..,"Dh":..,"Dv":..,"mask_heads":..,"causal":..},"plan":{"q":..,"k":..}};
// the reference's older whitespace-separated ten-integer lines and '#' comments are read as well.
// Measuring synchronises the host with the stream, so it is skipped while the stream is being captured.
#pragma once
#include <hip/hip_runtime.h>
#include <fcntl.h>
#include <stdint.h>
#include <sys/file.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/flame_attn.h"

namespace fattn {

struct PlanKey {
    int B, H, Q, K, Dh, Dv, mask_heads, causal;
    bool operator==(const PlanKey& o) const {
        return B == o.B && H == o.H && Q == o.Q && K == o.K && Dh == o.Dh && Dv == o.Dv && mask_heads == o.mask_heads &&
               causal == o.causal;
    }
};

struct PlanKeyHash {
    size_t operator()(const PlanKey& k) const {
        uint64_t h = 0xcbf29ce484222325ull;                  // FNV-1a over the eight fields
        for (int v : {k.B, k.H, k.Q, k.K, k.Dh, k.Dv, k.mask_heads, k.causal}) {
            h ^= (uint32_t)v;
            h *= 0x100000001b3ull;
        }
        return (size_t)h;
    }
};

struct Plan {
    int q_tile = 0, k_tile = 0;
    uint64_t last_used = 0;
};

enum PlanSource : uint64_t { kPlanNone = 0, kPlanCacheHit = 1, kPlanTuned = 2, kPlanRule = 3, kPlanForced = 4 };

struct PlanConfig {
    bool enabled = true, persist = false;
    int q_override = 0, warmups = 1, repeats = 3, flush_inserts = 200;
    double tie_eps = 0.02;
    size_t limit = 4096;
    std::string path;
};

inline int env_int(const char* name, int dflt) {
    const char* v = getenv(name);
    if (!v || !*v) return dflt;
    char* end = nullptr;
    const long x = strtol(v, &end, 10);
    return end == v ? dflt : (int)x;
}

inline bool env_flag(const char* name, bool dflt) {
    const char* v = getenv(name);
    if (!v || !*v) return dflt;
    const char c = (char)tolower((unsigned char)v[0]);
    if (c == '0' || c == 'f' || c == 'n') return false;
    if (c == '1' || c == 't' || c == 'y') return true;
    return dflt;
}

class PlanCache {
public:
    static PlanCache& instance() {
        static PlanCache* pc = new PlanCache;        // never destroyed: the exit handler below still needs it
        return *pc;
    }

    const PlanConfig& config() const { return cfg_; }

    // counters, under the lock
    template <class F>
    void with_stats(F&& f) {
        std::lock_guard<std::mutex> g(mu_);
        f(stats_);
    }

    bool lookup(const PlanKey& key, Plan* out) {
        std::lock_guard<std::mutex> g(mu_);
        load_locked();
        auto it = map_.find(key);
        if (it == map_.end()) return false;
        it->second.last_used = ++tick_;
        *out = it->second;
        return true;
    }

    void store(const PlanKey& key, int q_tile, int k_tile) {
        bool flush_now = false;
        {
            std::lock_guard<std::mutex> g(mu_);
            load_locked();
            if (meta_.empty()) meta_ = meta_line();      // now, while the device is certainly there (not at exit)
            const bool fresh = insert_locked(key, q_tile, k_tile);
            dirty_ = true;
            if (fresh && cfg_.persist && !cfg_.path.empty() && ++inserts_since_flush_ >= (size_t)cfg_.flush_inserts) flush_now = true;
        }
        if (flush_now) flush();
    }

    void get_stats(FlameSdpaAutotuneStats* out) {
        std::lock_guard<std::mutex> g(mu_);
        load_locked();
        stats_.cache_entries = map_.size();
        *out = stats_;
    }

    void reset_stats() {
        std::lock_guard<std::mutex> g(mu_);
        stats_ = FlameSdpaAutotuneStats{};
    }

    // Writes the cache to its file when persistence is on and something changed since the last write: entries
    // that another process added in the meantime are merged in first, the file is replaced atomically
    // (temporary file + rename) under an advisory lock.
    void flush() {
        std::lock_guard<std::mutex> g(mu_);
        load_locked();
        if (!cfg_.persist || cfg_.path.empty() || !dirty_) return;
        read_file_locked(false);
        if (!make_parent_dirs(cfg_.path)) return;
        const int lock_fd = ::open(cfg_.path.c_str(), O_RDWR | O_CREAT, 0644);
        if (lock_fd < 0) return;
        if (::flock(lock_fd, LOCK_EX | LOCK_NB) != 0) {
            ::close(lock_fd);
            return;
        }
        const std::string tmp = cfg_.path + ".tmp";
        bool ok = false;
        if (FILE* f = fopen(tmp.c_str(), "w")) {
            ok = fputs((meta_.empty() ? std::string("{\"meta\":{\"version\":1}}\n") : meta_).c_str(), f) >= 0;
            for (const auto& kv : map_) {
                const PlanKey& k = kv.first;
                ok = ok && fprintf(f, "{\"key\":{\"B\":%d,\"H\":%d,\"Q\":%d,\"K\":%d,\"Dh\":%d,\"Dv\":%d,\"mask_heads\":%d,\"causal\":%d},"
                                      "\"plan\":{\"q\":%d,\"k\":%d}}\n",
                                   k.B, k.H, k.Q, k.K, k.Dh, k.Dv, k.mask_heads, k.causal, kv.second.q_tile, kv.second.k_tile) > 0;
            }
            ok = ok && fflush(f) == 0 && fsync(fileno(f)) == 0;
            ok = (fclose(f) == 0) && ok;
        }
        if (ok && ::rename(tmp.c_str(), cfg_.path.c_str()) == 0) {
            dirty_ = false;
            inserts_since_flush_ = 0;
            stats_.cache_saved += 1;
        } else {
            ::unlink(tmp.c_str());
        }
        ::flock(lock_fd, LOCK_UN);
        ::close(lock_fd);
        stats_.cache_entries = map_.size();
    }

private:
    PlanCache() {
        cfg_.enabled = env_flag("FLAME_SDPA_AUTOTUNE", true);
        cfg_.q_override = std::max(0, env_int("FLAME_SDPA_QCHUNK", 0));
        cfg_.warmups = std::max(0, env_int("FLAME_SDPA_AUTOTUNE_WARMUPS", cfg_.warmups));
        cfg_.repeats = std::max(1, env_int("FLAME_SDPA_AUTOTUNE_REPEATS", cfg_.repeats));
        cfg_.tie_eps = std::max(0, env_int("FLAME_SDPA_AUTOTUNE_TIE_EPS_PCT", 2)) / 100.0;
        cfg_.persist = env_flag("FLAME_SDPA_AUTOTUNE_PERSIST", false);
        cfg_.flush_inserts = std::max(1, env_int("FLAME_SDPA_FLUSH_INSERTS", cfg_.flush_inserts));
        cfg_.limit = (size_t)std::max(1, env_int("FLAME_SDPA_AUTOTUNE_CACHE_LIMIT", (int)cfg_.limit));
        const char* p = getenv("FLAME_SDPA_AUTOTUNE_CACHE");
        if (p && *p) {
            cfg_.path = p;
        } else if (cfg_.persist) {
            const char* xdg = getenv("XDG_CACHE_HOME");
            const char* home = getenv("HOME");
            if (xdg && *xdg) cfg_.path = std::string(xdg) + "/flame/autotune_sdpa.json";
            else if (home && *home) cfg_.path = std::string(home) + "/.cache/flame/autotune_sdpa.json";
        }
        if (cfg_.persist && cfg_.path.empty()) cfg_.persist = false;
        if (cfg_.persist) atexit([] { PlanCache::instance().flush(); });
    }

    static bool make_parent_dirs(const std::string& file) {
        for (size_t pos = file.find('/', 1); pos != std::string::npos; pos = file.find('/', pos + 1)) {
            const std::string dir = file.substr(0, pos);
            if (::mkdir(dir.c_str(), 0755) != 0 && errno != EEXIST) return false;
        }
        return true;
    }

    static std::string meta_line() {
        int dev = -1, rt = 0;
        std::string arch = "unknown", name = "unknown";
        if (hipGetDevice(&dev) == hipSuccess) {
            hipDeviceProp_t prop;
            if (hipGetDeviceProperties(&prop, dev) == hipSuccess) {
                arch = prop.gcnArchName;
                name = prop.name;
            }
        } else {
            dev = -1;
            (void)hipGetLastError();
        }
        (void)hipRuntimeGetVersion(&rt);
        for (std::string* s : {&arch, &name})
            for (char& c : *s)
                if (c == '"' || c == '\\' || (unsigned char)c < 0x20) c = ' ';
        char buf[512];
        snprintf(buf, sizeof buf, "{\"meta\":{\"version\":1,\"device\":%d,\"arch\":\"%s\",\"runtime\":%d,\"name\":\"%s\"}}\n", dev,
                 arch.c_str(), rt, name.c_str());
        return buf;
    }

    // true when the key was not there before
    bool insert_locked(const PlanKey& key, int q_tile, int k_tile) {
        auto it = map_.find(key);
        const bool fresh = it == map_.end();
        Plan& p = map_[key];
        p.q_tile = q_tile;
        p.k_tile = k_tile;
        p.last_used = ++tick_;
        while (map_.size() > cfg_.limit) {                   // least recently used entry goes
            auto oldest = map_.begin();
            for (auto e = map_.begin(); e != map_.end(); ++e)
                if (e->second.last_used < oldest->second.last_used) oldest = e;
            map_.erase(oldest);
        }
        stats_.cache_entries = map_.size();
        return fresh;
    }

    static bool parse_line(std::string line, PlanKey* k, int* q, int* kt) {
        line.erase(std::remove_if(line.begin(), line.end(), [](unsigned char c) { return isspace(c); }), line.end());
        if (sscanf(line.c_str(),
                   "{\"key\":{\"B\":%d,\"H\":%d,\"Q\":%d,\"K\":%d,\"Dh\":%d,\"Dv\":%d,\"mask_heads\":%d,\"causal\":%d},\"plan\":{\"q\":%d,\"k\":%d}}",
                   &k->B, &k->H, &k->Q, &k->K, &k->Dh, &k->Dv, &k->mask_heads, &k->causal, q, kt) == 10)
            return true;
        return false;
    }

    void read_file_locked(bool count) {
        if (cfg_.path.empty()) return;
        FILE* f = fopen(cfg_.path.c_str(), "r");
        if (!f) return;
        if (count) stats_.cache_loads += 1;
        char buf[1024];
        bool version_ok = true;
        while (fgets(buf, sizeof buf, f)) {
            std::string line(buf);
            std::string compact = line;
            compact.erase(std::remove_if(compact.begin(), compact.end(), [](unsigned char c) { return isspace(c); }), compact.end());
            if (compact.empty() || compact[0] == '#') continue;
            if (compact.rfind("{\"meta\"", 0) == 0) {
                const size_t v = compact.find("\"version\":");
                if (v != std::string::npos && atol(compact.c_str() + v + 10) != 1) {
                    version_ok = false;
                    if (count) stats_.cache_load_errors += 1;
                }
                continue;
            }
            if (!version_ok) continue;
            PlanKey k{};
            int q = 0, kt = 0;
            bool ok = parse_line(line, &k, &q, &kt);
            if (!ok)      // the older format: ten integers separated by blanks
                ok = sscanf(line.c_str(), "%d %d %d %d %d %d %d %d %d %d", &k.B, &k.H, &k.Q, &k.K, &k.Dh, &k.Dv, &k.mask_heads,
                            &k.causal, &q, &kt) == 10;
            if (ok && q > 0 && kt > 0) {
                if (map_.find(k) == map_.end() || count) insert_locked(k, q, kt);       // a merge keeps what this process decided
            } else if (count) {
                stats_.cache_load_errors += 1;
            }
        }
        fclose(f);
        stats_.cache_entries = map_.size();
    }

    void load_locked() {
        if (loaded_) return;
        loaded_ = true;
        read_file_locked(cfg_.persist);
    }

    std::mutex mu_;
    PlanConfig cfg_;
    std::string meta_;
    std::unordered_map<PlanKey, Plan, PlanKeyHash> map_;
    FlameSdpaAutotuneStats stats_{};
    uint64_t tick_ = 0;
    size_t inserts_since_flush_ = 0;
    bool loaded_ = false, dirty_ = false;
};

}  // namespace fattn
