#include "handle.hpp"

#include <hip/hip_runtime_api.h>

namespace hipta
{
    namespace
    {
        struct Slot
        {
            uint64_t magic;
            Handle*  impl;
        };
    }

    Handle* Handle::create(int64_t* fields, int device, const std::string& arch, int cus, double clock_ghz)
    {
        Handle* h  = new Handle();
        h->mDevice = device;
        h->mArch   = arch;
        if(cus > 0)
            h->mModel.cus = cus;
        if(clock_ghz > 0)
            h->mModel.clock_ghz = clock_ghz;
        Slot* s  = reinterpret_cast<Slot*>(fields);
        s->magic = MAGIC;
        s->impl  = h;
        return h;
    }

    Handle* Handle::from(const int64_t* fields)
    {
        const Slot* s = reinterpret_cast<const Slot*>(fields);
        return s->magic == MAGIC ? s->impl : nullptr;
    }

    void Handle::destroy(int64_t* fields)
    {
        Slot* s = reinterpret_cast<Slot*>(fields);
        if(s->magic == MAGIC)
        {
            delete s->impl;
            s->magic = 0;
            s->impl  = nullptr;
        }
    }

    Handle::~Handle()
    {
        for(auto& kv : mPlans)
        {
            PlanState* p = kv.second.get();
            if(p && p->dev_block)
            {
                (void)hipFree(p->dev_block);
                p->dev_block = nullptr;
            }
            if(p)
                p->magic = 0;
        }
    }

    PlanState* Handle::intern(const std::string& key, std::unique_ptr<PlanState> fresh)
    {
        std::lock_guard<std::mutex> g(mLock);
        auto                        it = mPlans.find(key);
        if(it != mPlans.end())
        {
            if(fresh && fresh->dev_block)
                (void)hipFree(fresh->dev_block);
            return it->second.get();
        }
        PlanState* raw = fresh.get();
        mPlans.emplace(key, std::move(fresh));
        return raw;
    }

    PlanState* Handle::lookup(const std::string& key)
    {
        std::lock_guard<std::mutex> g(mLock);
        auto                        it = mPlans.find(key);
        return it == mPlans.end() ? nullptr : it->second.get();
    }

    size_t Handle::planCount()
    {
        std::lock_guard<std::mutex> g(mLock);
        return mPlans.size();
    }
}
