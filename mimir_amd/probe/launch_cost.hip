// What a dependent kernel launch costs on this device, taken apart: a stand-alone program (no part of
// the library) that replays chains of trivial kernels from a HIP graph and from a stream, and reports the
// period of a launch and how much of it lies inside the kernel (between the clock readings of its first
// and last instruction). The decoder's recorded step (llm/decode.go:79-160 in the reference; here a HIP
// graph of some 166 launches) is such a chain, so this fixed cost is what separates its speed from the
// sum of its kernels' work.
//
// Usage: launch_cost [nodes=200] [replays=20]
// Environment read by the HIP runtime before this program's first call, to be varied from outside:
//   HIP_FORCE_DEV_KERNARG=0|1   kernel arguments in host or device memory
// Compile-time variation: -mllvm -amdgpu-kernarg-preload-count=N (arguments preloaded into SGPRs).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#define CHECK(x)                                                                                   \
    do {                                                                                           \
        hipError_t e_ = (x);                                                                       \
        if (e_ != hipSuccess) {                                                                    \
            std::fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorName(e_)); \
            std::exit(1);                                                                          \
        }                                                                                          \
    } while (0)

// Every kernel leaves two readings of the 100 MHz clock in its slot: entry and exit of its first workgroup's
// first thread. slot == nullptr (k_none) leaves nothing.
struct Stamp {
    long long t_in, t_out;
};

__global__ void k_none() {}

__global__ __launch_bounds__(1024) void k_none_1024() {}

// reads its arguments (one trip to wherever they live) and stores
__global__ void k_stamp(Stamp* slot) {
    const long long t = wall_clock64();
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        slot->t_in = t;
        slot->t_out = wall_clock64();
    }
}

__global__ __launch_bounds__(1024) void k_stamp_1024(Stamp* slot) {
    const long long t = wall_clock64();
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        slot->t_in = t;
        slot->t_out = wall_clock64();
    }
}

// arguments, then one dependent load from device memory, as every real kernel starts
__global__ void k_load(Stamp* slot, const int* p) {
    const long long t = wall_clock64();
    const int v = *p;
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        slot->t_in = t;
        slot->t_out = wall_clock64() + (v == 0x7fffffff);
    }
}

// a kernarg segment of the decoder's products (some 220 bytes by value), the last field used
struct Fat {
    const int* p[26];
    int tail;
    int pad;
    Stamp* slot;
};
__global__ void k_fat(Fat f) {
    const long long t = wall_clock64();
    const int v = *f.p[25];
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        f.slot->t_in = t;
        f.slot->t_out = wall_clock64() + (v == 0x7fffffff) + (f.tail == 0x7fffffff);
    }
}

// the same job description resident in device memory, the kernel given its address
__global__ void k_fat_ptr(const Fat* f) {
    const long long t = wall_clock64();
    const int v = *f->p[25];
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        f->slot->t_in = t;
        f->slot->t_out = wall_clock64() + (v == 0x7fffffff) + (f->tail == 0x7fffffff);
    }
}

// a kernel that dirties n bytes (n / 4 threads store a dword each) before the next one starts
__global__ void k_write(Stamp* slot, int* out, int n4) {
    const long long t = wall_clock64();
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n4) out[i] = i;
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        slot->t_in = t;
        slot->t_out = wall_clock64();
    }
}

// a kernel that reads n bytes with 16-byte loads (NT: non-temporal ones) from every workgroup before the next one
// starts; its slot gets the first workgroup's entry and the last workgroup's exit
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
template <bool NT>
__global__ void k_read(Stamp* slot, const u32x4_t* src, long long n16, int* sink) {
    const long long t = wall_clock64();
    u32x4_t acc = {0, 0, 0, 0};
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (long long)gridDim.x * blockDim.x) {
        const u32x4_t v = NT ? __builtin_nontemporal_load(src + i) : src[i];
        acc ^= v;
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) sink[threadIdx.x] = 1;  // keeps the loads
    __syncthreads();
    if (threadIdx.x == 0) {
        if (blockIdx.x == 0) slot->t_in = t;
        atomicMax((unsigned long long*)&slot->t_out, (unsigned long long)wall_clock64());
    }
}

// a kernel with dynamic LDS
__global__ void k_lds(Stamp* slot) {
    extern __shared__ int lds[];
    const long long t = wall_clock64();
    lds[threadIdx.x] = (int)t;
    __syncthreads();
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        slot->t_in = t;
        slot->t_out = wall_clock64() + (lds[1] == 0x7fffffff);
    }
}

struct Launch {
    const char* name;
    int kind;  // 0 none, 1 none_1024, 2 stamp, 3 stamp_1024, 4 load, 5 fat, 6 fat_ptr, 7 write, 8 lds, 9 read, 10 read non-temporal
    int grid, block;
    int bytes;  // kind 7: bytes written; kind 8: dynamic LDS; kinds 9, 10: bytes read
};

struct Ctx {
    Stamp* stamps;
    int* word;
    int* sink;
    u32x4_t* big;  // 64 MB to read
    Fat* fat_dev;
    Fat fat_host;
};

static void launch(const Launch& l, Ctx& c, int node, hipStream_t st) {
    Stamp* slot = c.stamps + node;
    switch (l.kind) {
    case 0: hipLaunchKernelGGL(k_none, dim3(l.grid), dim3(l.block), 0, st); break;
    case 1: hipLaunchKernelGGL(k_none_1024, dim3(l.grid), dim3(l.block), 0, st); break;
    case 2: hipLaunchKernelGGL(k_stamp, dim3(l.grid), dim3(l.block), 0, st, slot); break;
    case 3: hipLaunchKernelGGL(k_stamp_1024, dim3(l.grid), dim3(l.block), 0, st, slot); break;
    case 4: hipLaunchKernelGGL(k_load, dim3(l.grid), dim3(l.block), 0, st, slot, (const int*)c.word); break;
    case 5: {
        Fat f = c.fat_host;
        f.slot = slot;
        hipLaunchKernelGGL(k_fat, dim3(l.grid), dim3(l.block), 0, st, f);
        break;
    }
    case 6: hipLaunchKernelGGL(k_fat_ptr, dim3(l.grid), dim3(l.block), 0, st, (const Fat*)(c.fat_dev + node)); break;
    case 7: hipLaunchKernelGGL(k_write, dim3((l.bytes / 4 + l.block - 1) / l.block), dim3(l.block), 0, st, slot, c.sink, l.bytes / 4); break;
    case 8: hipLaunchKernelGGL(k_lds, dim3(l.grid), dim3(l.block), l.bytes, st, slot); break;
    case 9: hipLaunchKernelGGL(k_read<false>, dim3(l.grid), dim3(l.block), 0, st, slot, (const u32x4_t*)c.big, (long long)l.bytes / 16, c.sink); break;
    case 10: hipLaunchKernelGGL(k_read<true>, dim3(l.grid), dim3(l.block), 0, st, slot, (const u32x4_t*)c.big, (long long)l.bytes / 16, c.sink); break;
    }
    CHECK(hipGetLastError());
}

struct Result {
    double graph_us, eager_us;  // period of one launch
    double inside_us;           // median t_out - t_in of the second kernel of the pattern (or the only one)
    double entry_gap_us;        // median of: this kernel's t_in minus the previous kernel's t_out
};

// A chain of `nodes` launches following `pattern` (one or two kinds alternating), from a graph and one by one.
static Result run(const std::vector<Launch>& pattern, Ctx& c, int nodes, int replays, hipStream_t st) {
    Result r{};
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    // eager
    for (int i = 0; i < nodes; i++) launch(pattern[i % pattern.size()], c, i, st);
    CHECK(hipStreamSynchronize(st));
    CHECK(hipEventRecord(e0, st));
    for (int rep = 0; rep < replays; rep++)
        for (int i = 0; i < nodes; i++) launch(pattern[i % pattern.size()], c, i, st);
    CHECK(hipEventRecord(e1, st));
    CHECK(hipStreamSynchronize(st));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    r.eager_us = ms * 1e3 / ((double)nodes * replays);
    // graph
    hipGraph_t g = nullptr;
    hipGraphExec_t ge = nullptr;
    CHECK(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
    for (int i = 0; i < nodes; i++) launch(pattern[i % pattern.size()], c, i, st);
    CHECK(hipStreamEndCapture(st, &g));
    CHECK(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0));
    CHECK(hipGraphLaunch(ge, st));
    CHECK(hipStreamSynchronize(st));
    CHECK(hipEventRecord(e0, st));
    for (int rep = 0; rep < replays; rep++) CHECK(hipGraphLaunch(ge, st));
    CHECK(hipEventRecord(e1, st));
    CHECK(hipStreamSynchronize(st));
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    r.graph_us = ms * 1e3 / ((double)nodes * replays);
    // the last replay's stamps
    const bool stamped = std::all_of(pattern.begin(), pattern.end(), [](const Launch& l) { return l.kind >= 2; });
    if (stamped) {
        std::vector<Stamp> h(nodes);
        CHECK(hipMemcpy(h.data(), c.stamps, sizeof(Stamp) * nodes, hipMemcpyDeviceToHost));
        std::vector<double> inside, gap;
        const int last = (int)pattern.size() - 1;
        for (int i = 8; i < nodes; i++) {
            if ((int)(i % pattern.size()) != last) continue;
            inside.push_back((h[i].t_out - h[i].t_in) / 100.0);
            gap.push_back((h[i].t_in - h[i - 1].t_out) / 100.0);
        }
        std::sort(inside.begin(), inside.end());
        std::sort(gap.begin(), gap.end());
        r.inside_us = inside[inside.size() / 2];
        r.entry_gap_us = gap[gap.size() / 2];
    } else {
        r.inside_us = r.entry_gap_us = -1;
    }
    CHECK(hipGraphExecDestroy(ge));
    CHECK(hipGraphDestroy(g));
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    return r;
}

int main(int argc, char** argv) {
    const int nodes = argc > 1 ? std::atoi(argv[1]) : 200;
    const int replays = argc > 2 ? std::atoi(argv[2]) : 20;
    if (nodes < 16 || nodes > 4096 || replays < 1 || replays > 1000) {
        std::fprintf(stderr, "launch_cost: nodes in 16..4096, replays in 1..1000\n");
        return 2;
    }
    CHECK(hipSetDevice(0));
    hipStream_t st;
    CHECK(hipStreamCreate(&st));
    Ctx c{};
    CHECK(hipMalloc(&c.stamps, sizeof(Stamp) * nodes));
    CHECK(hipMemset(c.stamps, 0, sizeof(Stamp) * nodes));
    CHECK(hipMalloc(&c.word, 256));
    CHECK(hipMemset(c.word, 0, 256));
    CHECK(hipMalloc(&c.sink, 4 << 20));
    CHECK(hipMalloc(&c.big, 64 << 20));
    CHECK(hipMemset(c.big, 1, 64 << 20));
    CHECK(hipMalloc(&c.fat_dev, sizeof(Fat) * nodes));
    for (int i = 0; i < 26; i++) c.fat_host.p[i] = c.word;
    c.fat_host.tail = 1;
    {
        std::vector<Fat> h(nodes, c.fat_host);
        for (int i = 0; i < nodes; i++) h[i].slot = c.stamps + i;
        CHECK(hipMemcpy(c.fat_dev, h.data(), sizeof(Fat) * nodes, hipMemcpyHostToDevice));
    }
    const char* env = std::getenv("HIP_FORCE_DEV_KERNARG");
#ifdef PRELOAD_NOTE
    const char* preload = PRELOAD_NOTE;
#else
    const char* preload = "none";
#endif
    std::printf("launch_cost: %d launches a chain, %d replays; HIP_FORCE_DEV_KERNARG=%s; kernarg preload: %s\n", nodes, replays, env ? env : "(unset)", preload);
    std::printf("| chain | graph us/launch | stream us/launch | inside kernel us | previous exit to entry us |\n|---|---|---|---|---|\n");
    struct Case {
        const char* name;
        std::vector<Launch> pattern;
    };
    const Launch none1{"none", 0, 1, 64, 0}, stamp1{"stamp", 2, 1, 64, 0};
    const std::vector<Case> cases = {
        {"no arguments, 1 x 64", {none1}},
        {"no arguments, 256 x 64", {{"none", 0, 256, 64, 0}}},
        {"no arguments, 256 x 1024 (launch bounds 1024)", {{"none", 1, 256, 1024, 0}}},
        {"no arguments, 2048 x 256", {{"none", 0, 2048, 256, 0}}},
        {"one pointer argument, stores 16 B, 1 x 64", {stamp1}},
        {"same, 256 x 64", {{"stamp", 2, 256, 64, 0}}},
        {"same, 256 x 1024", {{"stamp", 3, 256, 1024, 0}}},
        {"same, 2048 x 256", {{"stamp", 2, 2048, 256, 0}}},
        {"argument + one dependent load, 1 x 64", {{"load", 4, 1, 64, 0}}},
        {"same, 256 x 512", {{"load", 4, 256, 512, 0}}},
        {"224 B of arguments by value, last one used, 1 x 64", {{"fat", 5, 1, 64, 0}}},
        {"same, 256 x 512", {{"fat", 5, 256, 512, 0}}},
        {"the same 224 B behind one pointer (device memory), 1 x 64", {{"fatp", 6, 1, 64, 0}}},
        {"same, 256 x 512", {{"fatp", 6, 256, 512, 0}}},
        {"64 KB of dynamic LDS, 256 x 512", {{"lds", 8, 256, 512, 65536}}},
        {"1 KB of dynamic LDS, 256 x 512", {{"lds", 8, 256, 512, 1024}}},
        {"pair: a kernel that stores 16 B, then 1 x 64", {stamp1, stamp1}},
        {"pair: a kernel that stores 64 KB, then 1 x 64", {{"write", 7, 0, 256, 65536}, stamp1}},
        {"pair: a kernel that stores 1 MB, then 1 x 64", {{"write", 7, 0, 256, 1 << 20}, stamp1}},
        {"pair: a kernel that stores 4 MB, then 1 x 64", {{"write", 7, 0, 256, 4 << 20}, stamp1}},
        {"pair: 256 x 1024 stamps, then 1 x 64", {{"stamp", 3, 256, 1024, 0}, stamp1}},
        {"pair: 256 x 512 read 1 MB, then 1 x 64", {{"read", 9, 256, 512, 1 << 20}, stamp1}},
        {"pair: 256 x 512 read 33 MB, then 1 x 64", {{"read", 9, 256, 512, 33 << 20}, stamp1}},
        {"pair: the same 33 MB with non-temporal loads, then 1 x 64", {{"readnt", 10, 256, 512, 33 << 20}, stamp1}},
        {"pair: 256 x 512 read 33 MB, then 256 x 512 stamps", {{"read", 9, 256, 512, 33 << 20}, {"stamp", 2, 256, 512, 0}}},
    };
    for (const Case& cs : cases) {
        const Result r = run(cs.pattern, c, nodes, replays, st);
        const double per = cs.pattern.size();
        if (r.inside_us >= 0)
            std::printf("| %s | %.2f | %.2f | %.2f | %.2f |\n", cs.name, r.graph_us * per, r.eager_us * per, r.inside_us, r.entry_gap_us);
        else
            std::printf("| %s | %.2f | %.2f | - | - |\n", cs.name, r.graph_us * per, r.eager_us * per);
        std::fflush(stdout);
    }
    std::printf("(pairs: the period is of the pair; `inside` and `exit to entry` are of its second kernel)\n");
    return 0;
}
