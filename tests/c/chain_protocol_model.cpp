// A host-thread model of the hand-over inside the one-launch MLP (csrc/q4_chain.hip): producers
// (gate|up workgroups) publish tiles of h and count them on the counter of the 128-column step
// they belong to; consumers (down workgroups) ask a step's counter before they read the step.
// Counters are never reset: launch number n waits for 8 n.  Workgroups are handed to the places
// of their XCD in launch order, every consumer behind every producer, which is what the kernel's
// argument for freedom from deadlock rests on; the wait is bounded all the same.
//
// What the model checks, with few places per XCD so that workgroups really queue:
//   1. launch order: every launch ends, nobody gives up, every consumer read this launch's h;
//      tile counts that are not a multiple of 8 (the last step's extra), several launches on the
//      same counters, a change of the step count (counters zeroed, launch number back to 1);
//   2. the wrong order (consumers first, one place per XCD): consumers would wait for ever for
//      producers that cannot start - the bounded wait ends them, the launch reports that it gave
//      up, and the counters are still right for the next launch;
//   3. a withheld announcement (target one launch ahead): everyone gives up, the launch ends.
// Plain C++17 and std::thread; no GPU.  Prints "chain model ok" and exits 0, or says what failed.
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <random>
#include <thread>
#include <vector>

namespace {

constexpr uint32_t kTilesPerStep = 8;

struct Launch {
    uint32_t tiles;        // producer workgroups
    uint32_t steps;        // ceil(tiles / 8): counters in use
    uint32_t columns;      // consumer columns
    uint32_t slices;       // consumer rows: runs of steps
    uint32_t target;       // 8 * launch number
    uint32_t last_extra;   // 8 * steps - tiles
    uint32_t spin_limit;
    uint32_t epoch_tag;    // value producers write into h in this launch
};

struct Device {
    std::vector<std::atomic<uint32_t>> ready;
    std::vector<std::atomic<uint32_t>> h;  // one word per tile
    std::atomic<uint32_t> gave_up{0};
    std::atomic<uint32_t> stale_reads{0};
    explicit Device(size_t counters, size_t tiles) : ready(counters), h(tiles)
    {
        for (auto &c : ready) c.store(0);
        for (auto &t : h) t.store(0);
    }
};

void producer(Device &dev, const Launch &l, uint32_t tile, std::mt19937 &rng)
{
    std::this_thread::sleep_for(std::chrono::microseconds(rng() % 300));
    dev.h[tile].store(l.epoch_tag, std::memory_order_relaxed);
    // "outputs acknowledged, threads joined, then one count"
    const uint32_t add = 1u + (tile + 1u == l.tiles ? l.last_extra : 0u);
    dev.ready[tile / kTilesPerStep].fetch_add(add, std::memory_order_release);
}

void consumer(Device &dev, const Launch &l, uint32_t slice)
{
    const uint32_t slice_steps = (l.steps + l.slices - 1) / l.slices;
    const uint32_t begin = slice * slice_steps, end = std::min(l.steps, begin + slice_steps);
    bool asks = true;
    for (uint32_t step = begin; step < end; ++step) {
        if (asks) {
            uint32_t polls = 0;
            while ((int32_t)(dev.ready[step].load(std::memory_order_acquire) - l.target) < 0) {
                if (polls++ >= l.spin_limit) {
                    dev.gave_up.store(1);
                    asks = false;  // and never asks again
                    break;
                }
                std::this_thread::sleep_for(std::chrono::microseconds(20));
            }
        }
        for (uint32_t t = step * kTilesPerStep; t < std::min(l.tiles, (step + 1) * kTilesPerStep); ++t)
            if (dev.h[t].load(std::memory_order_relaxed) != l.epoch_tag) dev.stale_reads.fetch_add(1);
    }
}

// Runs one launch: workgroups [producers..., consumers...] (or the reverse) are dealt round-robin
// over `xcds` queues; each queue starts its workgroups in order as one of its `places` frees.
bool run_launch(Device &dev, const Launch &l, uint32_t xcds, uint32_t places, bool consumers_first, uint32_t seed)
{
    struct Work { bool produces; uint32_t index; };
    std::vector<Work> order;
    auto add_producers = [&] { for (uint32_t t = 0; t < l.tiles; ++t) order.push_back({true, t}); };
    auto add_consumers = [&] {
        for (uint32_t s = 0; s < l.slices; ++s)
            for (uint32_t c = 0; c < l.columns; ++c) order.push_back({false, s});
    };
    if (consumers_first) { add_consumers(); add_producers(); } else { add_producers(); add_consumers(); }
    std::vector<std::thread> queues;
    for (uint32_t x = 0; x < xcds; ++x) {
        queues.emplace_back([&, x] {
            std::mutex lock;
            std::condition_variable freed;
            uint32_t busy = 0;
            std::vector<std::thread> running;
            std::mt19937 rng(seed * 977u + x);
            for (size_t i = x; i < order.size(); i += xcds) {
                {
                    std::unique_lock<std::mutex> hold(lock);
                    freed.wait(hold, [&] { return busy < places; });
                    ++busy;
                }
                const Work w = order[i];
                const uint32_t sub_seed = (uint32_t)rng();
                running.emplace_back([&, w, sub_seed] {
                    std::mt19937 own(sub_seed);
                    if (w.produces) producer(dev, l, w.index, own); else consumer(dev, l, w.index);
                    { std::lock_guard<std::mutex> hold(lock); --busy; }
                    freed.notify_one();
                });
            }
            for (auto &t : running) t.join();
        });
    }
    for (auto &q : queues) q.join();
    return true;
}

Launch make_launch(uint32_t tiles, uint32_t columns, uint32_t slices, uint32_t number, uint32_t spin_limit, bool withhold)
{
    Launch l;
    l.tiles = tiles;
    l.steps = (tiles + kTilesPerStep - 1) / kTilesPerStep;
    l.columns = columns;
    l.slices = slices;
    l.target = kTilesPerStep * (number + (withhold ? 1u : 0u));
    l.last_extra = l.steps * kTilesPerStep - tiles;
    l.spin_limit = spin_limit;
    l.epoch_tag = 0x1000u + number;
    return l;
}

#define REQUIRE(condition, ...)                                   \
    do {                                                          \
        if (!(condition)) {                                       \
            fprintf(stderr, "chain model: " __VA_ARGS__);         \
            fprintf(stderr, "\n");                                \
            return 1;                                             \
        }                                                         \
    } while (0)

}  // namespace

int main()
{
    // 1. launch order, few places: tiles 44 (not a multiple of 8), three slices, five launches
    {
        Device dev(64, 64);
        uint32_t number = 0;
        for (int launch = 0; launch < 5; ++launch) {
            const Launch l = make_launch(44, 6, 3, ++number, 1u << 20, false);
            run_launch(dev, l, 4, 2, false, 10 + launch);
            REQUIRE(dev.gave_up.load() == 0, "launch %d in order gave up", launch);
            REQUIRE(dev.stale_reads.load() == 0, "launch %d read %u stale tiles", launch, dev.stale_reads.load());
            for (uint32_t s = 0; s < l.steps; ++s)
                REQUIRE(dev.ready[s].load() == l.target, "counter %u is %u after launch %u", s, dev.ready[s].load(), number);
        }
        // another step count: the host zeroes the counters and starts numbering again
        for (auto &c : dev.ready) c.store(0);
        number = 0;
        for (int launch = 0; launch < 3; ++launch) {
            const Launch l = make_launch(17, 3, 2, ++number, 1u << 20, false);
            run_launch(dev, l, 4, 1, false, 30 + launch);
            REQUIRE(dev.gave_up.load() == 0 && dev.stale_reads.load() == 0, "second shape, launch %d", launch);
        }
    }
    // 2. the wrong order with one place per XCD: bounded waits end it, and it says so
    {
        Device dev(64, 64);
        const Launch l = make_launch(24, 4, 1, 1, 50, false);
        run_launch(dev, l, 2, 1, true, 77);
        REQUIRE(dev.gave_up.load() == 1, "consumers in front of producers did not give up");
        for (uint32_t s = 0; s < l.steps; ++s)
            REQUIRE(dev.ready[s].load() == l.target, "counter %u wrong after the abandoned launch", s);
        dev.gave_up.store(0);
        dev.stale_reads.store(0);
        const Launch next = make_launch(24, 4, 1, 2, 1u << 20, false);
        run_launch(dev, next, 2, 1, false, 78);
        REQUIRE(dev.gave_up.load() == 0 && dev.stale_reads.load() == 0, "launch after the abandoned one");
    }
    // 3. withheld announcement: everyone gives up, the launch ends, the next one is right
    {
        Device dev(64, 64);
        const Launch l = make_launch(32, 4, 2, 1, 20, true);
        run_launch(dev, l, 4, 3, false, 5);
        REQUIRE(dev.gave_up.load() == 1, "withheld launch did not give up");
        dev.gave_up.store(0);
        dev.stale_reads.store(0);
        const Launch next = make_launch(32, 4, 2, 2, 1u << 20, false);
        run_launch(dev, next, 4, 3, false, 6);
        REQUIRE(dev.gave_up.load() == 0 && dev.stale_reads.load() == 0, "launch after the withheld one");
    }
    printf("chain model ok\n");
    return 0;
}
