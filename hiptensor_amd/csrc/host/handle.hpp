// Library context stored inside hiptensorHandle_t::fields, and the immutable plan
// state a hiptensorContractionPlan_t points at.
//
// Reference counterparts: Handle / HipDevice (library/src/handle.cpp:31-60,
// library/src/hip_device.cpp:32-78).  Differences by design: gfx950 is the one
// accepted architecture (the reference exits the process on it), device properties
// are read once per handle rather than on every call, and the handle owns every plan
// state it created, because the API has no call that destroys a plan.
#pragma once
#include <atomic>
#include <cstdint>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "hiptk_kernels.h"
#include "planner.hpp"
#include "repack.hpp"
#include "solution.hpp"

namespace hipta
{
    struct PlanState
    {
        uint64_t        magic = 0;
        GemmView        view; // host copy of the folded problem (tables kept for inspection)
        hiptk_problem_t prob{}; // table pointers are device addresses (null on a host-only handle)
        const Solution* sol       = nullptr;
        uint64_t        ws_bytes  = 0; // workspace the plan needs: packed copies, then split-K partials
        PackedOperand   pack_a, pack_b; // operands moved into a packed copy before the kernel runs
        uint64_t        pack_bytes = 0; // leading part of the workspace that holds those copies
        void*           dev_block = nullptr; // one allocation holding all eight tables
        int             device    = -1;
        int             compute   = 0; // hiptensorComputeType_t (how alpha / beta are read)
        std::string     kernel_name;
        double          est_us = 0.0;
        // last planning or execution that touched this state (a process-wide tick): the handle's
        // cache retires the least recently used state when it is full
        mutable std::atomic<uint64_t> last_use{0};
        // Set, under the owning handle's lock, by the first execution of a plan made from this state.
        // From then on the device may hold the table addresses beyond the call (a captured graph
        // replays them, another thread may be between its checks and its launch), so the cache never
        // retires such a state: it lives until hiptensorDestroy.  Only states that were planned and
        // never executed are candidates for retirement.
        mutable std::atomic<bool> launched{false};
        class Handle*             owner = nullptr;
        static constexpr uint64_t MAGIC   = 0x504c414e68697074ull;
        // a state whose device tables were released: its handle was destroyed, or the handle's cache
        // retired it.  The (small) object itself stays allocated until the process ends, so a plan
        // that still points at it is refused instead of reading freed memory.
        static constexpr uint64_t RETIRED = 0x5245544952454421ull;
    };

    uint64_t next_use_tick();

    class Handle
    {
    public:
        static constexpr uint64_t MAGIC = 0x48444c4568697074ull;

        // Places a Handle behind the 4 KiB blob; device < 0 creates a host-only handle
        // (planning and inspection work, execution is refused).
        static Handle* create(int64_t* fields, int device, const std::string& arch, int cus, double clock_ghz);
        static Handle* from(const int64_t* fields);
        static void    destroy(int64_t* fields);

        int                device() const { return mDevice; }
        bool               hostOnly() const { return mDevice < 0; }
        const DeviceModel& model() const { return mModel; }
        const std::string& arch() const { return mArch; }

        // The cache has two levels.  A *request* key names what the caller asked for (problem,
        // algorithm, workspace size, overrides); a *decision* key names what planning made of it
        // (problem, kernel, split-K, packed copies).  Many requests (e.g. every workspace size) share
        // one decision, and only decisions own a PlanState and device tables: their number is bounded
        // by the kernel registry, not by the values callers pass.
        PlanState* lookup(const std::string& request);
        PlanState* findDecision(const std::string& request, const std::string& decision);
        // Adopts `fresh` under `decision` (or returns the state another thread adopted first, freeing
        // fresh's device block) and remembers `request` as an alias of it.
        PlanState* intern(const std::string& request, const std::string& decision, std::unique_ptr<PlanState> fresh);
        // To be called by every execution before it uses `st`: false if the state was retired (its
        // handle destroyed, or the cache dropped it before any execution); otherwise the state is
        // marked as launched and stays valid until its handle is destroyed.
        static bool pin(const PlanState* st);
        size_t     planCount();
        size_t     aliasCount();
        // most states / aliases a handle keeps (HIPTENSOR_AMD_PLAN_CACHE=<states> overrides the first);
        // states that have been executed do not count as removable, so a handle that executes more
        // distinct plans than this keeps them all
        static constexpr size_t MAX_PLANS   = 4096;
        static constexpr size_t MAX_ALIASES = 16384;

    private:
        Handle() = default;
        ~Handle();
        int                                               mDevice = -1;
        std::string                                       mArch;
        DeviceModel                                       mModel;
        std::mutex                                        mLock;
        std::map<std::string, std::unique_ptr<PlanState>> mPlans; // by decision key
        std::map<std::string, PlanState*>                 mAlias; // request key -> state
        size_t                                            mMaxPlans = MAX_PLANS;
        void retire(std::unique_ptr<PlanState> p); // releases the device tables, keeps the header
        void alias(const std::string& request, PlanState* st);
    };
}
