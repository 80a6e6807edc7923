// Host-side exercise of the kvmove C ABI under AddressSanitizer / UBSan (host code only; no
// GPU is needed and none is touched).  Walks every argument-checking path that returns
// before a launch, with index lists large and small, malformed geometry, bad handles and
// the divider arithmetic, and checks the error codes.  Built and run by
// tests/test_host_sanitize.py; exits non-zero on a wrong code (the sanitizers abort on
// their own findings).
#include "kvmove.h"

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

static int failures = 0;
#define EXPECT(cond)                                                        \
    do {                                                                    \
        if (!(cond)) {                                                      \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);   \
            ++failures;                                                     \
        }                                                                   \
    } while (0)

static KvmGeom geom(int64_t L, int64_t H, int64_t B, int64_t D, int64_t s, int cpp = 1, int ctp = 1, int dpp = 1,
                    int dtp = 1, int q = 0, int u = 0)
{
    KvmGeom g;
    std::memset(&g, 0, sizeof g);
    g.num_layers = L; g.num_kv_heads = H; g.block_size = B; g.head_dim = D; g.dtype_bytes = s;
    g.ctx_pp_size = cpp; g.ctx_tp_size = ctp; g.dec_pp_size = dpp; g.dec_tp_size = dtp;
    g.dec_pp_rank = q; g.dec_tp_rank = u;
    return g;
}

int main()
{
    EXPECT(kvm_version() / 10000 == KVM_ABI_MAJOR);
    EXPECT(std::strlen(kvm_last_error()) == 0);

    // options: every name, valid and invalid values, unknown and null names
    const char *names[] = {"swap_mode", "swap_wgs", "swap_wgs_in", "swap_kernel_below", "xcd_map", "sort_pairs"};
    for (const char *n : names) {
        const int64_t old = kvm_get_option(n);
        EXPECT(kvm_set_option(n, old) == KVM_OK);
        EXPECT(kvm_set_option(n, -7) == KVM_EINVAL);
        EXPECT(kvm_get_option(n) == old);
    }
    EXPECT(kvm_set_option("no_such_option", 1) == KVM_EINVAL);
    EXPECT(kvm_set_option("threads", 64) == KVM_EINVAL);        // a knob of the exploration build only
    EXPECT(kvm_set_option(nullptr, 1) == KVM_EINVAL);
    EXPECT(kvm_get_option(nullptr) == KVM_EINVAL);
    EXPECT(std::strlen(kvm_last_error()) > 0);

    // geometry and argument validation of kvm_migrate (returns before any HIP call)
    char fake_k[64], fake_v[64];
    std::vector<int64_t> ci(2000), di(2000);
    std::mt19937_64 rng(5);
    for (size_t i = 0; i < ci.size(); ++i) { ci[i] = (int64_t)(rng() % 64); di[i] = (int64_t)i; }
    KvmGeom g = geom(4, 4, 16, 8, 2);
    EXPECT(kvm_migrate(nullptr, ci.data(), di.data(), 1, fake_k, fake_v, 8, nullptr) == KVM_EINVAL);
    EXPECT(kvm_migrate(&g, ci.data(), di.data(), -1, fake_k, fake_v, 8, nullptr) == KVM_EINVAL);
    EXPECT(kvm_migrate(&g, ci.data(), di.data(), 1, nullptr, fake_v, 8, nullptr) == KVM_EINVAL);
    EXPECT(kvm_migrate(&g, ci.data(), di.data(), 1, fake_k, fake_v, 0, nullptr) == KVM_EINVAL);
    EXPECT(kvm_migrate(&g, nullptr, di.data(), 1, fake_k, fake_v, 8, nullptr) == KVM_EINVAL);
    EXPECT(kvm_migrate(&g, ci.data(), di.data(), 2000, fake_k, fake_v, 4096, nullptr) == KVM_ENOTREG);
    KvmGeom bad = geom(5, 4, 16, 8, 2, 2);
    EXPECT(kvm_migrate(&bad, ci.data(), di.data(), 1, fake_k, fake_v, 8, nullptr) == KVM_EINVAL);
    bad = geom(4, 6, 16, 8, 2, 1, 4);
    EXPECT(kvm_migrate(&bad, ci.data(), di.data(), 1, fake_k, fake_v, 8, nullptr) == KVM_EINVAL);
    bad = geom(4, 4, 0, 8, 2);
    EXPECT(kvm_migrate(&bad, ci.data(), di.data(), 1, fake_k, fake_v, 8, nullptr) == KVM_EINVAL);
    bad = geom(4, 4, 16, 8, 2, 1, 1, 2, 2, 2, 0);
    EXPECT(kvm_migrate(&bad, ci.data(), di.data(), 1, fake_k, fake_v, 8, nullptr) == KVM_EINVAL);
    bad = geom(1 << 20, 1 << 10, 16, 128, 2);                   // a block beyond 4 GiB
    EXPECT(kvm_migrate(&bad, ci.data(), di.data(), 1, fake_k, fake_v, 8, nullptr) == KVM_EINVAL);
    int64_t plan[10];
    EXPECT(kvm_migrate_plan(&g, 10, fake_k, fake_v, 64, nullptr) == KVM_EINVAL);
    EXPECT(kvm_migrate_plan(&g, 10, fake_k, fake_v, 64, plan) == KVM_ENOTREG);
    KvmGeom other = g;
    other.ctx_instance = 3;                                     // no instance has anything registered
    EXPECT(kvm_migrate_plan(&other, 10, fake_k, fake_v, 64, plan) == KVM_ENOTREG);

    // Launch sizes, as pure arithmetic (null pools: nothing registered, no device touched).
    // A launch is 2 * tiles * blocks workgroups of 64 lanes and must stay below 2^32 work-items,
    // so big blocks get fewer index pairs per launch instead of a launch the runtime refuses.
    EXPECT(kvm_migrate_plan(&g, -1, nullptr, nullptr, 0, plan) == KVM_EINVAL);
    {
        // LLaMA-2-7B 1 -> 1: 4 MiB per pool kind per block = 4096 tiles; 432 blocks per launch out of
        // pools of unknown size, 864 when every pool has at most 65536 blocks
        KvmGeom g7 = geom(32, 32, 16, 128, 2);
        EXPECT(kvm_migrate_plan(&g7, 909, nullptr, nullptr, 0, plan) == KVM_OK);
        EXPECT(plan[0] == 8192 && plan[1] == 64 && plan[2] == 16 && plan[3] == 1 && plan[4] == 3 && plan[6] == 1);
        EXPECT(plan[5] == 8388608);
        EXPECT(plan[7] == 2ll * 4096 * 432 * 64 && plan[8] == 1 && plan[9] == 432);
        EXPECT(kvm_migrate_plan(&g7, 909, nullptr, nullptr, 4096, plan) == KVM_OK);
        EXPECT(plan[4] == 2 && plan[7] == 2ll * 4096 * 864 * 64 && plan[9] == 864);
        EXPECT(kvm_migrate_plan(&g7, 909, nullptr, nullptr, 65537, plan) == KVM_OK && plan[9] == 432);
        // pp4 x tp4 context ranks feed one decoding rank: 16 segments = 2 groups of 8, and 900 pairs are
        // 2 launches per group of 864 packed pairs (3 of 432 wide ones)
        KvmGeom g16 = geom(8, 8, 16, 8, 2, 4, 4);
        EXPECT(kvm_migrate_plan(&g16, 900, nullptr, nullptr, 1024, plan) == KVM_OK);
        EXPECT(plan[3] == 16 && plan[4] == 4 && plan[6] == 0);
        EXPECT(kvm_migrate_plan(&g16, 900, nullptr, nullptr, 0, plan) == KVM_OK && plan[4] == 6);
        // a 1 GiB block per pool kind (L 128 x H 128 x B 256 x D 128 x 2 bytes): 2^20 tiles, so at
        // most 31 blocks fit a launch (2 * 31 * 2^20 * 64 < 2^32 <= 2 * 32 * 2^20 * 64)
        KvmGeom big = geom(128, 128, 256, 128, 2);
        for (int64_t n : {1, 31, 32, 100, 432, 1000}) {
            EXPECT(kvm_migrate_plan(&big, n, nullptr, nullptr, 4096, plan) == KVM_OK);
            EXPECT(plan[5] == 2ll << 30);
            EXPECT(plan[7] > 0 && plan[7] < (1ll << 32));
            EXPECT(plan[4] == (n + 30) / 31);
            EXPECT(plan[7] == 2ll * (1 << 20) * (n < 31 ? n : 31) * 64);
        }
        // the same through two context ranks whose head split does not nest (general kernel, 2 segments)
        KvmGeom big2 = geom(128, 128, 256, 128, 2, 1, 2);
        EXPECT(kvm_migrate_plan(&big2, 100, nullptr, nullptr, 4096, plan) == KVM_OK);
        EXPECT(plan[3] == 2 && plan[6] == 0 && plan[7] < (1ll << 32) && plan[4] == 4);
        // many small blocks: every launch of 432 (or 864) pairs is far below the limit
        KvmGeom small = geom(2, 2, 16, 8, 2);
        EXPECT(kvm_migrate_plan(&small, 100000, nullptr, nullptr, 100000, plan) == KVM_OK);
        EXPECT(plan[4] == (100000 + 431) / 432 && plan[7] < (1ll << 32));
        EXPECT(kvm_migrate_plan(&small, 60000, nullptr, nullptr, 65536, plan) == KVM_OK);
        EXPECT(plan[4] == (60000 + 863) / 864 && plan[7] < (1ll << 32));
    }

    // handles and registration
    int64_t h[KVM_HANDLE_WORDS] = {0};
    int64_t pc[4] = {1, 0, 1, 0}, bad_pc[4] = {1, 3, 1, 0};
    EXPECT(kvm_get_mem_handle(nullptr, 16, h) == KVM_EINVAL);
    EXPECT(kvm_get_mem_handle(fake_k, 0, h) == KVM_EINVAL);
    EXPECT(kvm_get_mem_handle(fake_k, 16, nullptr) == KVM_EINVAL);
    EXPECT(kvm_get_mem_handle(fake_k, 16, h) == KVM_EINVAL);    // host memory (or no device at all) is no pool
    EXPECT(kvm_register_mem_handle(h, h, 4, 4, pc, pc, 0) == KVM_EHANDLE);
    EXPECT(kvm_register_mem_handle(nullptr, h, 4, 4, pc, pc, 0) == KVM_EINVAL);
    EXPECT(kvm_register_mem_handle(h, h, 4, 4, nullptr, pc, 0) == KVM_EINVAL);
    EXPECT(kvm_register_mem_handle(h, h, 4, 4, pc, bad_pc, 0) == KVM_EINVAL);
    h[0] = 0x4b564d4f56453034LL; h[1] = 1; h[2] = 0; h[3] = 4096; h[4] = 64;   // plausible but forged: checksum missing
    EXPECT(kvm_register_mem_handle(h, h, 4, 4, pc, pc, 0) == KVM_EHANDLE);
    EXPECT(std::strstr(kvm_last_error(), "not a kvmove memory handle") != nullptr);
    // well-formed handles of another process (pid 1), with the checksum word as the library computes it
    auto seal = [](int64_t *w) {
        uint64_t x = 0x5a5a5a5a5a5a5a5aull;
        for (int i = 0; i < KVM_HANDLE_WORDS - 1; ++i) x = ((x << 7) | (x >> 57)) ^ (uint64_t)w[i];
        w[KVM_HANDLE_WORDS - 1] = (int64_t)x;
    };
    h[5] = 4096; h[6] = 1 << 20; h[7] = 0;                      // made without an IPC part
    seal(h);
    EXPECT(kvm_register_mem_handle(h, h, 4, 4, pc, pc, 0) == KVM_EHANDLE);
    EXPECT(std::strstr(kvm_last_error(), "was not exported for other processes") != nullptr);
    h[6] = 3ll << 30;                                           // inside a 3 GiB allocation: never shared
    seal(h);
    EXPECT(kvm_register_mem_handle(h, h, 4, 4, pc, pc, 0) == KVM_EHANDLE);
    EXPECT(std::strstr(kvm_last_error(), "are not shared between processes") != nullptr);
    h[7] = 1;                                                   // claims an IPC part all the same
    seal(h);
    EXPECT(kvm_register_mem_handle(h, h, 4, 4, pc, pc, 0) == KVM_EHANDLE);
    EXPECT(std::strstr(kvm_last_error(), "inconsistent") != nullptr);
    h[6] = 32;                                                  // pool of 64 bytes in an allocation of 32
    seal(h);
    EXPECT(kvm_register_mem_handle(h, h, 4, 4, pc, pc, 0) == KVM_EHANDLE);
    EXPECT(std::strstr(kvm_last_error(), "inconsistent") != nullptr);
    h[5] = 8192;                                                // pool below its allocation
    h[6] = 1 << 20;
    seal(h);
    EXPECT(kvm_register_mem_handle(h, h, 4, 4, pc, pc, 0) == KVM_EHANDLE);
    EXPECT(std::strstr(kvm_last_error(), "inconsistent") != nullptr);
    h[4] = 0;                                                   // names no memory
    seal(h);
    EXPECT(kvm_register_mem_handle(h, h, 4, 4, pc, pc, 0) == KVM_EHANDLE);
    EXPECT(kvm_opened_handles() == 0);
    EXPECT(kvm_register_source(1, 1, 0, 0, 4, 4, nullptr, fake_v, 64, 0) == KVM_EINVAL);
    EXPECT(kvm_register_source(1, 1, 1, 0, 4, 4, fake_k, fake_v, 64, 0) == KVM_EINVAL);
    EXPECT(kvm_register_source(2, 1, 0, 0, 5, 4, fake_k, fake_v, 64, 0) == KVM_EINVAL);
    EXPECT(kvm_register_source(1, 1, 0, 0, 4, 4, fake_k, fake_v, 64, 7) == KVM_EINVAL);   // not device memory
    EXPECT(kvm_reset() == KVM_OK);

    // swap and plain copy argument checks
    EXPECT(kvm_swap(ci.data(), di.data(), 1, 1, nullptr, fake_v, fake_k, fake_v, 64, 4, 4, nullptr) == KVM_EINVAL);
    EXPECT(kvm_swap(ci.data(), di.data(), -1, 1, fake_k, fake_v, fake_k, fake_v, 64, 4, 4, nullptr) == KVM_EINVAL);
    EXPECT(kvm_swap(ci.data(), di.data(), 1, 0, fake_k, fake_v, fake_k, fake_v, 0, 4, 4, nullptr) == KVM_EINVAL);
    EXPECT(kvm_swap(ci.data(), di.data(), 1, 0, fake_k, fake_v, fake_k, fake_v, 64, 0, 4, nullptr) == KVM_EINVAL);
    EXPECT(kvm_swap(ci.data(), di.data(), 1, 0, fake_k, fake_v, fake_k, fake_v, 64, 4, 4, nullptr) == KVM_EINVAL);
    EXPECT(kvm_copy_plain(nullptr, fake_k, 16, nullptr) == KVM_EINVAL);
    EXPECT(kvm_copy_plain(fake_k, fake_v, -1, nullptr) == KVM_EINVAL);
    EXPECT(kvm_copy_plain(fake_k, fake_v, 0, nullptr) == KVM_OK);

    EXPECT(kvm_copy_plain(fake_k, fake_v, 16, nullptr) == KVM_EINVAL);   // not device memory

    // the swap plan touches no device: run lists of many shapes through it
    int64_t sp[4];
    EXPECT(kvm_swap_plan(ci.data(), di.data(), 1, 64, 0, 0, 0, nullptr) == KVM_EINVAL);
    EXPECT(kvm_swap_plan(nullptr, di.data(), 1, 64, 0, 0, 0, sp) == KVM_EINVAL);
    EXPECT(kvm_swap_plan(ci.data(), di.data(), 1, 0, 0, 0, 0, sp) == KVM_EINVAL);
    EXPECT(kvm_swap_plan(nullptr, nullptr, 0, 64, 0, 0, 0, sp) == KVM_OK && sp[1] == 0);
    // the default takes the copy kernel whatever the slab size, with its own workgroup count per direction
    EXPECT(kvm_swap_plan(ci.data(), di.data(), 5, 4 << 20, 0, 0, 0, sp) == KVM_OK && sp[0] == 1 && sp[3] == kvm_get_option("swap_wgs"));
    EXPECT(kvm_swap_plan(ci.data(), di.data(), 5, 4 << 20, 1, 0, 0, sp) == KVM_OK && sp[0] == 1 && sp[3] == kvm_get_option("swap_wgs_in"));
    // with a threshold, large copies go to the copy engines as before
    EXPECT(kvm_set_option("swap_kernel_below", 2 << 20) == KVM_OK);
    for (int round = 0; round < 200; ++round) {
        const int64_t n = (int64_t)(rng() % 3000);
        std::vector<int64_t> a((size_t)n), b((size_t)n);
        int64_t runs = n > 0 ? 1 : 0;
        for (int64_t i = 0; i < n; ++i) {
            const bool follow = i > 0 && rng() % 3 != 0;
            a[(size_t)i] = follow ? a[(size_t)i - 1] + 1 : (int64_t)(rng() % 100000);
            b[(size_t)i] = follow ? b[(size_t)i - 1] + 1 : (int64_t)(rng() % 100000);
            if (i > 0 && !(a[(size_t)i] == a[(size_t)i - 1] + 1 && b[(size_t)i] == b[(size_t)i - 1] + 1)) ++runs;
        }
        const int64_t slab = (int64_t)1 << (rng() % 24);
        // pools of 100000 blocks (ids up to there) need wide pairs; every third round plans for small pools
        const bool small_pools = round % 3 == 0;
        EXPECT(kvm_swap_plan(a.data(), b.data(), n, slab, round & 1, small_pools ? 65536 : 200000,
                             small_pools ? 4096 : 200000, sp) == KVM_OK);
        EXPECT(sp[1] == runs);
        const int64_t want = runs > 0 && n * slab / runs < (2 << 20) ? 1 : 2;
        EXPECT(sp[0] == want);
        const int64_t per = small_pools ? 864 : 432;
        EXPECT(sp[2] == (want == 1 ? (n + per - 1) / per : 0));
        if (failures) break;
    }
    EXPECT(kvm_set_option("swap_kernel_below", 1ll << 32) == KVM_OK);

    // the divider arithmetic, many operands
    for (int i = 0; i < 200000; ++i) {
        const uint32_t d = (uint32_t)(rng() >> (rng() % 40)) | 1u;
        const uint32_t n = (uint32_t)rng();
        EXPECT(kvm_debug_divide(n, d) == n / d);
        if (failures) break;
    }
    EXPECT(kvm_debug_divide(7, 0) == UINT32_MAX);

    if (failures) {
        std::printf("%d check(s) failed\n", failures);
        return 1;
    }
    std::printf("abi_sanitize: all checks passed\n");
    return 0;
}
