// Host-side bookkeeping for kernels that hand work over between workgroups through arrival counters held in a
// file-scope __device__ array (the one-launch beam top-K, the few-row projection kernel cut along K, the built-in
// scratch of onellm_decode_attn_static).  One policy for all of them:
//
//   * the array is cut into sets; a set belongs to one (device, workspace pointer) from the first launch that uses
//     that workspace until the caller gives it back with onellm_release_workspace().  A set never changes hands on
//     its own - not when the table is full, not after any time - because a launch recorded into a graph keeps the
//     counters it was given for as long as the graph lives, and a call on another stream may be in flight;
//   * when every set of a device is owned, acquire() returns -1: the caller runs its counter-free form (a second
//     launch, an uncut run, the GEMM library) and reports that through its *_last_path query; the table counts such
//     calls (onellm_counter_set_fallbacks) and says so on stderr once;
//   * counters are zero when the module is loaded and every kernel that uses a set leaves it at zero, so a set
//     needs no clearing when it is handed out or given back.
//
// Header-only on purpose: the table is plain host logic (testable without a GPU); only the process-wide list that
// onellm_release_workspace walks lives in libonellm_hip.so (counter_sets.cpp).
#pragma once
#include <stdio.h>
#include <map>
#include <mutex>
#include <vector>

namespace onellm {

class CounterSets;
// the process-wide list of tables onellm_release_workspace / onellm_counter_set_fallbacks walk (libonellm_hip.so)
void counter_sets_register(CounterSets* table);
void counter_sets_unregister(CounterSets* table);

class CounterSets {
public:
    // `what` names the table in the one-line notice; `listed`: put the table on the process-wide list
    CounterSets(const char* what, int sets_per_device, bool listed = true)
        : what_(what), nsets_(sets_per_device), listed_(listed)
    {
        if (listed_) counter_sets_register(this);
    }
    ~CounterSets()
    {
        if (listed_) counter_sets_unregister(this);
    }
    CounterSets(const CounterSets&) = delete;
    CounterSets& operator=(const CounterSets&) = delete;

    // The set of `workspace` on `device`: the one it owns, else a free one (which it owns from now on), else -1.
    // `capturing`: the launch is being recorded into a graph - remembered, so that stats can tell how many sets
    // replays may use at any time.
    int acquire(int device, const void* workspace, bool capturing = false)
    {
        std::lock_guard<std::mutex> lock(mu_);
        std::vector<Owner>& sets = per_device_[device];
        if (sets.empty()) sets.resize((size_t)nsets_);
        int free_set = -1;
        for (int i = 0; i < nsets_; ++i) {
            if (sets[(size_t)i].workspace == workspace && sets[(size_t)i].owned) {
                sets[(size_t)i].captured = sets[(size_t)i].captured || capturing;
                return i;
            }
            if (free_set < 0 && !sets[(size_t)i].owned) free_set = i;
        }
        if (free_set < 0) {
            ++fallbacks_;
            if (!told_) {
                told_ = true;
                fprintf(stderr, "[oneLLM][WARN] %s: all %d counter sets of device %d belong to other workspaces; this call "
                                "runs its form without counters (slower).  Give the sets of workspaces that are no longer "
                                "used back with onellm_release_workspace().\n", what_, nsets_, device);
            }
            return -1;
        }
        sets[(size_t)free_set] = Owner{workspace, true, capturing};
        return free_set;
    }

    // Gives back every set `workspace` owns (on any device).  The caller states that no launch that was handed this
    // workspace is queued, running, or recorded in a graph that will be replayed.  Returns how many sets were freed.
    int release(const void* workspace)
    {
        std::lock_guard<std::mutex> lock(mu_);
        int n = 0;
        for (auto& dev : per_device_)
            for (Owner& o : dev.second)
                if (o.owned && o.workspace == workspace) {
                    o = Owner{};
                    ++n;
                }
        return n;
    }

    struct Stats {
        int owned, captured;
        long fallbacks;
    };
    Stats stats(int device)
    {
        std::lock_guard<std::mutex> lock(mu_);
        Stats s{0, 0, fallbacks_};
        auto it = per_device_.find(device);
        if (it != per_device_.end())
            for (const Owner& o : it->second) {
                s.owned += o.owned ? 1 : 0;
                s.captured += (o.owned && o.captured) ? 1 : 0;
            }
        return s;
    }
    long fallbacks()
    {
        std::lock_guard<std::mutex> lock(mu_);
        return fallbacks_;
    }
    int sets_per_device() const { return nsets_; }

private:
    struct Owner {
        const void* workspace = nullptr;
        bool owned = false;
        bool captured = false;
    };
    const char* what_;
    const int nsets_;
    const bool listed_;
    std::mutex mu_;
    std::map<int, std::vector<Owner>> per_device_;
    long fallbacks_ = 0;
    bool told_ = false;
};

}  // namespace onellm
