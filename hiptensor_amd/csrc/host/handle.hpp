// Library context stored inside hiptensorHandle_t::fields, and the immutable plan
// state a hiptensorContractionPlan_t points at.
//
// Reference counterparts: Handle / HipDevice (library/src/handle.cpp:31-60,
// library/src/hip_device.cpp:32-78).  Differences by design: gfx950 is the one
// accepted architecture (the reference exits the process on it), device properties
// are read once per handle rather than on every call, and the handle owns every plan
// state it created, because the API has no call that destroys a plan.
#pragma once
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
        static constexpr uint64_t MAGIC = 0x504c414e68697074ull;
    };

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

        // Returns the cached state for `key`, or adopts `fresh` under that key.
        PlanState* intern(const std::string& key, std::unique_ptr<PlanState> fresh);
        PlanState* lookup(const std::string& key);
        size_t     planCount();

    private:
        Handle() = default;
        ~Handle();
        int                                               mDevice = -1;
        std::string                                       mArch;
        DeviceModel                                       mModel;
        std::mutex                                        mLock;
        std::map<std::string, std::unique_ptr<PlanState>> mPlans;
    };
}
