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
    EXPECT(kvm_version() >= 100);
    EXPECT(std::strlen(kvm_last_error()) == 0);

    // options: every name, valid and invalid values, unknown and null names
    const char *names[] = {"tile_bytes", "threads", "unroll", "nt_load", "nt_store", "swap_mode", "swap_wgs",
                           "lds_pad", "wave_contig", "xcd_map", "simple"};
    for (const char *n : names) {
        const int64_t old = kvm_get_option(n);
        EXPECT(kvm_set_option(n, old) == KVM_OK);
        EXPECT(kvm_set_option(n, -7) == KVM_EINVAL);
        EXPECT(kvm_get_option(n) == old);
    }
    EXPECT(kvm_set_option("no_such_option", 1) == KVM_EINVAL);
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
    int64_t plan[8];
    EXPECT(kvm_migrate_plan(&g, 10, fake_k, fake_v, nullptr) == KVM_EINVAL);
    EXPECT(kvm_migrate_plan(&g, 10, fake_k, fake_v, plan) == KVM_ENOTREG);

    // handles and registration
    int64_t h[KVM_HANDLE_WORDS] = {0};
    int64_t pc[4] = {1, 0, 1, 0}, bad_pc[4] = {1, 3, 1, 0};
    EXPECT(kvm_get_mem_handle(nullptr, 16, h) == KVM_EINVAL);
    EXPECT(kvm_get_mem_handle(fake_k, 0, h) == KVM_EINVAL);
    EXPECT(kvm_get_mem_handle(fake_k, 16, nullptr) == KVM_EINVAL);
    EXPECT(kvm_get_mem_handle(fake_k, 16, h) == KVM_EINVAL);    // host memory (or no device at all) is no pool
    EXPECT(kvm_register_mem_handle(h, h, 4, 4, pc, pc) == KVM_EHANDLE);
    EXPECT(kvm_register_mem_handle(nullptr, h, 4, 4, pc, pc) == KVM_EINVAL);
    EXPECT(kvm_register_mem_handle(h, h, 4, 4, nullptr, pc) == KVM_EINVAL);
    h[0] = 0x4b564d4f56453031LL; h[1] = 1; h[2] = 0; h[3] = 4096; h[4] = 64;   // plausible but forged: checksum missing
    EXPECT(kvm_register_mem_handle(h, h, 4, 4, pc, pc) == KVM_EHANDLE);
    h[5] = h[0] ^ h[1] ^ h[2] ^ h[3] ^ h[4];                                   // well formed, other process (pid 1)
    EXPECT(kvm_register_mem_handle(h, h, 4, 4, pc, pc) == KVM_EHANDLE);
    (void)bad_pc;
    EXPECT(kvm_register_source(1, 1, 0, 0, 4, 4, nullptr, fake_v, 64) == KVM_EINVAL);
    EXPECT(kvm_register_source(1, 1, 1, 0, 4, 4, fake_k, fake_v, 64) == KVM_EINVAL);
    EXPECT(kvm_register_source(2, 1, 0, 0, 5, 4, fake_k, fake_v, 64) == KVM_EINVAL);
    EXPECT(kvm_register_source(1, 1, 0, 0, 4, 4, fake_k, fake_v, 64) == KVM_EINVAL);   // not device memory
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
    EXPECT(kvm_swap_plan(ci.data(), di.data(), 1, 64, nullptr) == KVM_EINVAL);
    EXPECT(kvm_swap_plan(nullptr, di.data(), 1, 64, sp) == KVM_EINVAL);
    EXPECT(kvm_swap_plan(ci.data(), di.data(), 1, 0, sp) == KVM_EINVAL);
    EXPECT(kvm_swap_plan(nullptr, nullptr, 0, 64, sp) == KVM_OK && sp[1] == 0);
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
        EXPECT(kvm_swap_plan(a.data(), b.data(), n, slab, sp) == KVM_OK);
        EXPECT(sp[1] == runs);
        const int64_t want = runs > 0 && n * slab / runs < (2 << 20) ? 1 : 2;
        EXPECT(sp[0] == want);
        EXPECT(sp[2] == (want == 1 ? (n + 431) / 432 : 0));
        if (failures) break;
    }

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
