#include "handle.hpp"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdlib>
#include <iterator>

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
        if(const char* e = std::getenv("HIPTENSOR_AMD_PLAN_CACHE"))
            h->mMaxPlans = (size_t)std::max(1, std::atoi(e));
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

    namespace
    {
        std::atomic<uint64_t> g_tick{1};
        // retired plan states: kept (a few hundred bytes each) so that a stale plan reads RETIRED
        std::mutex                              g_graveyard_lock;
        std::vector<std::unique_ptr<PlanState>> g_graveyard;
    }

    uint64_t next_use_tick()
    {
        return g_tick.fetch_add(1, std::memory_order_relaxed);
    }

    void Handle::retire(std::unique_ptr<PlanState> p)
    {
        if(!p)
            return;
        if(p->dev_block)
        {
            (void)hipFree(p->dev_block);
            p->dev_block = nullptr;
        }
        p->prob  = hiptk_problem_t{};
        p->magic = PlanState::RETIRED;
        for(std::vector<int32_t>* t : {&p->view.xp, &p->view.xk, &p->view.yq, &p->view.yk, &p->view.cp, &p->view.cq, &p->view.dp, &p->view.dq})
            std::vector<int32_t>().swap(*t);
        std::lock_guard<std::mutex> g(g_graveyard_lock);
        g_graveyard.push_back(std::move(p));
    }

    Handle::~Handle()
    {
        for(auto& kv : mPlans)
            retire(std::move(kv.second));
        mPlans.clear();
        mAlias.clear();
    }

    void Handle::alias(const std::string& request, PlanState* st)
    {
        if(mAlias.size() >= MAX_ALIASES)
            mAlias.clear(); // aliases only save a re-planning on the host
        mAlias[request] = st;
    }

    PlanState* Handle::lookup(const std::string& request)
    {
        std::lock_guard<std::mutex> g(mLock);
        auto                        it = mAlias.find(request);
        if(it == mAlias.end())
            return nullptr;
        it->second->last_use.store(next_use_tick(), std::memory_order_relaxed);
        return it->second;
    }

    PlanState* Handle::findDecision(const std::string& request, const std::string& decision)
    {
        std::lock_guard<std::mutex> g(mLock);
        auto                        it = mPlans.find(decision);
        if(it == mPlans.end())
            return nullptr;
        it->second->last_use.store(next_use_tick(), std::memory_order_relaxed);
        alias(request, it->second.get());
        return it->second.get();
    }

    PlanState* Handle::intern(const std::string& request, const std::string& decision, std::unique_ptr<PlanState> fresh)
    {
        std::unique_ptr<PlanState> victim;
        PlanState*                 raw = nullptr;
        {
            std::lock_guard<std::mutex> g(mLock);
            auto                        it = mPlans.find(decision);
            if(it != mPlans.end())
            {
                if(fresh && fresh->dev_block)
                    (void)hipFree(fresh->dev_block);
                alias(request, it->second.get());
                return it->second.get();
            }
            if(mPlans.size() >= mMaxPlans)
            {
                // retire the least recently planned state among those that were never executed (an
                // executed state's tables may still be read by the device: a captured graph, a launch
                // in another thread); if every state has been executed the cache grows instead
                auto lru = mPlans.end();
                for(auto jt = mPlans.begin(); jt != mPlans.end(); ++jt)
                {
                    if(jt->second->launched.load(std::memory_order_acquire))
                        continue;
                    if(lru == mPlans.end()
                       || jt->second->last_use.load(std::memory_order_relaxed) < lru->second->last_use.load(std::memory_order_relaxed))
                        lru = jt;
                }
                if(lru != mPlans.end())
                {
                    for(auto at = mAlias.begin(); at != mAlias.end();)
                        at = at->second == lru->second.get() ? mAlias.erase(at) : std::next(at);
                    victim        = std::move(lru->second);
                    victim->magic = PlanState::RETIRED; // under the lock: pin() refuses it from here on
                    mPlans.erase(lru);
                }
            }
            raw        = fresh.get();
            raw->owner = this;
            raw->last_use.store(next_use_tick(), std::memory_order_relaxed);
            mPlans.emplace(decision, std::move(fresh));
            alias(request, raw);
        }
        retire(std::move(victim));
        return raw;
    }

    bool Handle::pin(const PlanState* st)
    {
        // (retired states stay allocated for the life of the process, so these reads are safe)
        if(!st || st->magic != PlanState::MAGIC)
            return false;
        if(st->launched.load(std::memory_order_acquire))
            return true;
        Handle* o = st->owner;
        if(!o)
            return false;
        // the cache retires states under this lock: either it has retired this one already, or it
        // sees the mark and leaves it alone
        std::lock_guard<std::mutex> g(o->mLock);
        if(st->magic != PlanState::MAGIC)
            return false;
        st->launched.store(true, std::memory_order_release);
        return true;
    }

    size_t Handle::planCount()
    {
        std::lock_guard<std::mutex> g(mLock);
        return mPlans.size();
    }

    size_t Handle::aliasCount()
    {
        std::lock_guard<std::mutex> g(mLock);
        return mAlias.size();
    }
}
