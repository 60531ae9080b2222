// Host-only check of include/qm_attn.hpp: the adapters must throw std::runtime_error exactly
// where the reference's launch wrappers and overflow guards do.  No device call is reached.
#include <cstdio>
#include <cstring>
#include <string>

#include "../include/qm_attn.hpp"

static int failures = 0;

template <class F>
static void expect_throw(const char* what, const char* needle, F f) {
    try {
        f();
        std::printf("FAIL %s: no exception\n", what);
        ++failures;
    } catch (const std::runtime_error& e) {
        if (!std::strstr(e.what(), needle)) {
            std::printf("FAIL %s: message '%s' lacks '%s'\n", what, e.what(), needle);
            ++failures;
        } else {
            std::printf("ok   %s: %s\n", what, e.what());
        }
    }
}

int main() {
    auto* fake = reinterpret_cast<std::uint16_t*>(0x10000);
    expect_throw("append overflow", "cache overflow", [&] {
        qm_attn::launch_qk_norm_rope_cache_m1(fake, fake, fake, fake, fake, fake, fake, fake, fake, fake, 16, 8, 128,
                                              2061, 2061, 1e-6f, nullptr);
    });
    expect_throw("append null", "pointer is NULL", [&] {
        qm_attn::launch_qk_norm_rope_cache_m1(nullptr, fake, fake, fake, fake, fake, fake, fake, fake, fake, 16, 8,
                                              128, 64, 3, 1e-6f, nullptr);
    });
    expect_throw("append head_dim", "geometry", [&] {
        qm_attn::launch_qk_norm_rope_cache_m1(fake, fake, fake, fake, fake, fake, fake, fake, fake, fake, 16, 8, 64,
                                              64, 3, 1e-6f, nullptr);
    });
    expect_throw("attention overflow", "capacity", [&] {
        qm_attn::launch_attention(fake, fake, fake, fake, 1, 64, 16, 8, 128, 64, -1, 0.088f, nullptr, 0, nullptr);
    });
    expect_throw("attention group", "geometry", [&] {
        qm_attn::launch_attention(fake, fake, fake, fake, 1, 10, 20, 8, 128, 64, -1, 0.088f, nullptr, 0, nullptr);
    });
    expect_throw("attention workspace", "workspace", [&] {
        qm_attn::launch_attention(fake, fake, fake, fake, 1, 8000, 16, 8, 128, 8206, -1, 0.088f, nullptr, 0, nullptr);
    });
    expect_throw("chunked prefill overflow", "cache overflow", [&] {
        qm_attn::launch_attention(fake, fake, fake, fake, 8, 60, 16, 8, 128, 64, -1, 0.088f, nullptr, 0, nullptr);
    });
    expect_throw("windowed rows workspace", "workspace", [&] {
        qm_attn::launch_attention(fake, fake, fake, fake, 8, 1000, 16, 8, 128, 2048, 512, 0.088f, nullptr, 0, nullptr);
    });
    expect_throw("chunked prefill group", "geometry", [&] {
        qm_attn::launch_attention(fake, fake, fake, fake, 8, 5, 20, 8, 128, 64, -1, 0.088f, nullptr, 0, nullptr);
    });
    expect_throw("scatter decode overflow", "cache overflow", [&] {
        qm_attn::scatter_decode_cache(fake, fake, fake, fake, 8, 128, 64, 64, nullptr);
    });
    expect_throw("scatter prefill overflow", "capacity", [&] {
        qm_attn::scatter_prefill_cache(fake, fake, fake, fake, 65, 8, 128, 64, nullptr);
    });
    expect_throw("predictor key_length", "key_length", [&] {
        qm_attn::predictor_attention_m1(fake, fake, fake, fake, 17, nullptr);
    });
    expect_throw("predictor loop rows", "invalid argument", [&] {
        qm_attn::predictor_attention_loop(fake, fake, fake, fake, fake, fake, fake, fake, nullptr, nullptr, 1, 5, 17, 1,
                                          1e-6f, nullptr);
    });
    expect_throw("predictor update_cache overflow", "capacity", [&] {
        qm_attn::predictor_update_cache(fake, fake, 2, 15, nullptr);
    });
    expect_throw("predictor rope null", "pointer is NULL", [&] {
        qm_attn::predictor_rope(fake, nullptr, fake, fake, 2, 16, nullptr);
    });
    if (qm_attn::attention_workspace_bytes(16, 8, 8206) == 0) {
        std::printf("FAIL workspace size is zero for a long context\n");
        ++failures;
    }
    std::printf("%d failure(s)\n", failures);
    return failures ? 1 : 0;
}
