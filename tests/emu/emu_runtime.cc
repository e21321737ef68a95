// Execution engine of the CPU emulation build (see hip/hip_runtime.h in this directory): test infrastructure only.
//
// A launch runs workgroup after workgroup.  A workgroup first runs its lanes one after the other on the calling
// thread, from the last lane to the first: the one cross-lane operation the kernels use hands lane i a value of
// lane i + 1, which has then already run and left that value in a log.  The first lane that reaches a barrier
// cannot go on alone: it unwinds (an exception), and the workgroup, and every later workgroup of the launch, runs
// again from the start with one OS thread per lane.  No kernel of the library stores to global memory before its
// first barrier, so the part of a workgroup that ran twice wrote nothing the second run reads.
#include <hip/hip_runtime.h>

#include <condition_variable>
#include <mutex>
#include <thread>
#include <vector>

namespace hccl_amd {
namespace detail {
// The dynamic LDS of the reduce kernel (`extern __shared__ uint32_t accStack[]`): the whole 160 KiB of a CU.
uint32_t accStack[160 * 1024 / 4];
}  // namespace detail
}  // namespace hccl_amd

namespace emu {

thread_local Idx tIdx = {0, 0, 0};
thread_local Idx bIdx = {0, 0, 0};
Idx gDim = {1, 1, 1};
Idx bDim = {1, 1, 1};

namespace {

struct NeedsLockstep {};

// A barrier whose party may shrink: a lane that has left the kernel is no longer waited for, as on the GPU.
class Barrier {
public:
    void Reset(unsigned parties)
    {
        std::lock_guard<std::mutex> g(mu_);
        parties_ = parties;
        waiting_ = 0;
    }
    void Wait()
    {
        std::unique_lock<std::mutex> g(mu_);
        const uint64_t gen = gen_;
        if (++waiting_ >= parties_) {
            waiting_ = 0;
            ++gen_;
            cv_.notify_all();
            return;
        }
        cv_.wait(g, [&] { return gen_ != gen; });
    }
    void Leave()
    {
        std::lock_guard<std::mutex> g(mu_);
        --parties_;
        if (parties_ != 0 && waiting_ >= parties_) {
            waiting_ = 0;
            ++gen_;
            cv_.notify_all();
        }
    }

private:
    std::mutex mu_;
    std::condition_variable cv_;
    unsigned parties_ = 0;
    unsigned waiting_ = 0;
    uint64_t gen_ = 0;
};

constexpr unsigned kWave = 64;
thread_local bool t_lockstep = false;   // this OS thread is one lane of a workgroup that runs in lockstep mode
thread_local unsigned t_flat = 0;       // flat index of the lane in its workgroup

struct Group {
    Barrier all;
    std::vector<Barrier> wave;
    std::vector<uint32_t> exchange;   // one word per lane, for WaveShl1
};
Group* g_group = nullptr;
// Sequential mode: the values every lane of the workgroup in progress has passed to WaveShl1, call by call.
std::vector<std::vector<uint32_t>> g_shlLog;
unsigned g_seqLane = 0;

Idx LaneIdx(unsigned flat, const dim3& block)
{
    return Idx{flat % block.x, (flat / block.x) % block.y, flat / (block.x * block.y)};
}

// Lanes of lockstep workgroups run on a pool of OS threads that lives as long as the process: worker t runs lane t
// of every workgroup that has more than t lanes.  Starting threads per workgroup would cost far more than the work.
class Pool {
public:
    void Run(unsigned lanes, const dim3& block, const Idx& blk, const std::function<void()>& body, Group* group)
    {
        std::unique_lock<std::mutex> g(mu_);
        while (workers_.size() < lanes) {
            const unsigned t = static_cast<unsigned>(workers_.size());
            workers_.emplace_back([this, t] { Work(t); });
            workers_.back().detach();
        }
        lanes_ = lanes;
        block_ = block;
        blk_ = blk;
        body_ = &body;
        group_ = group;
        running_ = lanes;
        ++epoch_;
        start_.notify_all();
        done_.wait(g, [&] { return running_ == 0; });
    }

private:
    void Work(unsigned t)
    {
        uint64_t seen = 0;
        std::unique_lock<std::mutex> g(mu_);
        for (;;) {
            start_.wait(g, [&] { return epoch_ != seen; });
            seen = epoch_;
            if (t >= lanes_) {
                continue;
            }
            const std::function<void()>* body = body_;
            Group* group = group_;
            tIdx = LaneIdx(t, block_);
            bIdx = blk_;
            t_lockstep = true;
            t_flat = t;
            g.unlock();
            (*body)();
            group->all.Leave();
            group->wave[t / kWave].Leave();
            g.lock();
            if (--running_ == 0) {
                done_.notify_all();
            }
        }
    }

    std::mutex mu_;
    std::condition_variable start_, done_;
    std::vector<std::thread> workers_;
    uint64_t epoch_ = 0;
    unsigned lanes_ = 0;
    unsigned running_ = 0;
    dim3 block_;
    Idx blk_ = {0, 0, 0};
    const std::function<void()>* body_ = nullptr;
    Group* group_ = nullptr;
};

void RunLockstep(unsigned lanes, const dim3& block, const Idx& blk, const std::function<void()>& body)
{
    static Pool* pool = new Pool;   // never destroyed: its threads outlive main
    Group group;
    const unsigned waves = (lanes + kWave - 1) / kWave;
    group.all.Reset(lanes);
    group.wave = std::vector<Barrier>(waves);
    for (unsigned w = 0; w < waves; ++w) {
        const unsigned inWave = (w + 1) * kWave <= lanes ? kWave : lanes - w * kWave;
        group.wave[w].Reset(inWave);
    }
    group.exchange.assign(lanes, 0);
    g_group = &group;
    pool->Run(lanes, block, blk, body, &group);
    g_group = nullptr;
}

}  // namespace

void SyncThreads()
{
    if (!t_lockstep) {
        throw NeedsLockstep{};
    }
    g_group->all.Wait();
}

uint32_t WaveShl1(uint32_t old, uint32_t src)
{
    if (!t_lockstep) {
        // Lanes run in descending order: the right-hand neighbour has finished, its k-th value is in the log.  A
        // neighbour that made fewer calls was inactive at this one, and the lane keeps `old` as on the GPU.
        const unsigned lane = g_seqLane;
        const size_t k = g_shlLog[lane].size();
        g_shlLog[lane].push_back(src);
        const bool lastOfWave = (lane % kWave) == kWave - 1 || lane + 1 >= g_shlLog.size();
        return (lastOfWave || g_shlLog[lane + 1].size() <= k) ? old : g_shlLog[lane + 1][k];
    }
    Group& g = *g_group;
    const unsigned lanes = static_cast<unsigned>(g.exchange.size());
    Barrier& wave = g.wave[t_flat / kWave];
    g.exchange[t_flat] = src;
    wave.Wait();
    const bool last = (t_flat % kWave) == kWave - 1 || t_flat + 1 >= lanes;
    const uint32_t got = last ? old : g.exchange[t_flat + 1];
    wave.Wait();
    return got;
}

void Launch(dim3 grid, dim3 block, const std::function<void()>& body)
{
    // One launch at a time: the library serialises its launches per world, tests may run several worlds.
    static std::mutex launchMu;
    std::lock_guard<std::mutex> guard(launchMu);
    gDim = Idx{grid.x, grid.y, grid.z};
    bDim = Idx{block.x, block.y, block.z};
    const unsigned lanes = block.x * block.y * block.z;
    const Idx savedT = tIdx;
    const Idx savedB = bIdx;
    bool lockstep = false;
    for (unsigned bz = 0; bz < grid.z; ++bz) {
        for (unsigned by = 0; by < grid.y; ++by) {
            for (unsigned bx = 0; bx < grid.x; ++bx) {
                const Idx blk{bx, by, bz};
                if (!lockstep) {
                    try {
                        bIdx = blk;
                        g_shlLog.resize(lanes);
                        for (std::vector<uint32_t>& log : g_shlLog) {
                            log.clear();
                        }
                        for (unsigned t = lanes; t-- > 0;) {
                            tIdx = LaneIdx(t, block);
                            g_seqLane = t;
                            body();
                        }
                        continue;
                    } catch (const NeedsLockstep&) {
                        lockstep = true;
                    }
                }
                RunLockstep(lanes, block, blk, body);
            }
        }
    }
    tIdx = savedT;
    bIdx = savedB;
}

}  // namespace emu
