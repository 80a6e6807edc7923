// Host-side exercise of the kvmove C ABI's locks under ThreadSanitizer (host code only; no GPU
// is needed and none is touched).  Several threads plan migrations (which walks the registry
// under its shared lock), set and read options, register forged handles of "another process"
// (refused before anything is mapped), and reset, all at once; every call must return the code
// it returns alone, and each thread's error text must be its own.  Built and run by
// tests/test_host_sanitize.py; exits non-zero on a wrong code (the sanitizer reports races itself).
#include "kvmove.h"

#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <thread>
#include <vector>

static std::atomic<int> failures{0};
#define EXPECT(cond)                                                        \
    do {                                                                    \
        if (!(cond)) {                                                      \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);   \
            ++failures;                                                     \
        }                                                                   \
    } while (0)

static KvmGeom geom(int64_t L, int64_t H, int cpp, int ctp)
{
    KvmGeom g;
    std::memset(&g, 0, sizeof g);
    g.num_layers = L; g.num_kv_heads = H; g.block_size = 16; g.head_dim = 128; g.dtype_bytes = 2;
    g.ctx_pp_size = cpp; g.ctx_tp_size = ctp; g.dec_pp_size = 1; g.dec_tp_size = 1;
    return g;
}

int main()
{
    const int kRounds = 2000;
    std::vector<std::thread> threads;
    // planners: pure arithmetic under the registry's shared lock
    for (int t = 0; t < 3; ++t)
        threads.emplace_back([t] {
            for (int i = 0; i < kRounds; ++i) {
                KvmGeom g = geom(32, 32, 1 + (i + t) % 2, 1 << (i % 4));
                int64_t plan[10];
                EXPECT(kvm_migrate_plan(&g, 100 + i % 900, nullptr, nullptr, 4096, plan) == KVM_OK);
                EXPECT(plan[9] == 864 && plan[4] >= 1 && plan[7] < (1ll << 32));
                KvmGeom bad = geom(33, 32, 2, 1);
                EXPECT(kvm_migrate_plan(&bad, 1, nullptr, nullptr, 4096, plan) == KVM_EINVAL);
                EXPECT(std::strstr(kvm_last_error(), "not divisible") != nullptr);   // this thread's own text
            }
        });
    // option writers and readers
    threads.emplace_back([] {
        for (int i = 0; i < kRounds; ++i) {
            EXPECT(kvm_set_option("swap_wgs", 8 + i % 16) == KVM_OK);
            const int64_t v = kvm_get_option("swap_wgs");
            EXPECT(v >= 8 && v < 24);
            EXPECT(kvm_set_option("sort_pairs", i % 3) == KVM_OK);
            EXPECT(kvm_set_option("no_such_option", 1) == KVM_EINVAL);
            EXPECT(std::strstr(kvm_last_error(), "unknown option") != nullptr);
        }
        EXPECT(kvm_set_option("swap_wgs", 16) == KVM_OK && kvm_set_option("sort_pairs", 1) == KVM_OK);
    });
    // registrations that are refused before anything is mapped, and resets
    threads.emplace_back([] {
        int64_t h[KVM_HANDLE_WORDS] = {0};
        int64_t pc[4] = {1, 0, 1, 0};
        for (int i = 0; i < kRounds; ++i) {
            EXPECT(kvm_register_mem_handle(h, h, 4, 4, pc, pc, i % 3) == KVM_EHANDLE);
            EXPECT(std::strstr(kvm_last_error(), "not a kvmove memory handle") != nullptr);
            if (i % 50 == 0) EXPECT(kvm_reset() == KVM_OK);
            EXPECT(kvm_opened_handles() == 0);
        }
    });
    // swap plans: no lock, thread-local scratch
    threads.emplace_back([] {
        std::vector<int64_t> a(3000), b(3000);
        for (size_t i = 0; i < a.size(); ++i) { a[i] = (int64_t)(i * 7 % 4096); b[i] = (int64_t)i; }
        int64_t sp[4];
        for (int i = 0; i < kRounds; ++i) {
            EXPECT(kvm_swap_plan(a.data(), b.data(), 1 + i % 3000, 4 << 20, i & 1, 4096, 4096, sp) == KVM_OK);
            EXPECT(sp[0] == 1 && sp[2] == (1 + i % 3000 + 863) / 864);
        }
    });
    for (std::thread &t : threads) t.join();
    if (failures.load()) {
        std::printf("%d check(s) failed\n", failures.load());
        return 1;
    }
    std::printf("abi_threads: all checks passed\n");
    return 0;
}
