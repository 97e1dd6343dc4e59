// Host-side rules under AddressSanitizer + UndefinedBehaviorSanitizer.
//
// Built by tests/test_host_sanitizers.py with g++ -fsanitize=address,undefined from this file,
// ratchet_amd/csrc/spec.cpp and ratchet_amd/csrc/gguf.cpp (-DRT_HOST_ONLY: no HIP), and run on
//   - the GGUF images named on the command line, whole, truncated at every length, and with
//     seeded byte and 8-byte-word corruptions (hostile counts, lengths, offsets, types), each parsed,
//     walked through every accessor, and every tensor's byte range asked for;
//   - a grid of Matmul descriptors (ranks 0..5, extents including 0 and 2^62, every dtype id
//     in and out of range, every flag combination) through validate / infer / make_spec.
// Any sanitizer report aborts the process; the driver itself only checks that failures are
// statuses.  Exit code 0 and the line "ok" mean a clean run.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "../ratchet_amd/csrc/spec.h"

struct rt_gguf;
namespace rt {
rt_status gguf_tensor_range(const rt_gguf *g, uint64_t size, uint64_t index, uint64_t *begin, uint64_t *numel_out, std::string &why);
}

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static uint64_t rnd() { // splitmix64
    uint64_t z = (rng_state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static long n_ok = 0, n_err = 0, n_ranges = 0, n_range_err = 0;

static void walk(const uint8_t *img, uint64_t size) {
    // the image is copied into an exactly-sized heap block so that any read past it is seen
    uint8_t *buf = (uint8_t *)malloc(size ? size : 1);
    if (size) memcpy(buf, img, size);
    rt_gguf *g = nullptr;
    const rt_status st = rt_gguf_parse(buf, size, &g);
    if (st != RT_OK) {
        if (g) { fprintf(stderr, "handle returned with an error status\n"); exit(2); }
        n_err++;
        free(buf);
        return;
    }
    n_ok++;
    (void)rt_gguf_version(g);
    (void)rt_gguf_error(g);
    const uint64_t nt = rt_gguf_tensor_count(g), nk = rt_gguf_metadata_count(g);
    for (uint64_t i = 0; i <= nk; i++) { // one past the end on purpose
        const char *key = nullptr;
        if (rt_gguf_metadata_key_at(g, i, &key) != RT_OK) continue;
        rt_gguf_value v;
        if (rt_gguf_metadata_get(g, key, &v) == RT_OK && v.type == RT_GGUF_ARRAY) {
            rt_gguf_value e;
            for (uint64_t j = 0; j <= v.count && j < 64; j++) (void)rt_gguf_metadata_array_get(g, key, j, &e);
            (void)rt_gguf_metadata_array_get(g, key, v.count, &e);
            (void)rt_gguf_metadata_array_get(g, key, UINT64_MAX, &e);
        }
        if (v.type == RT_GGUF_STRING && v.str) (void)strlen(v.str);
    }
    rt_gguf_value v;
    (void)rt_gguf_metadata_get(g, "no.such.key", &v);
    for (uint64_t i = 0; i <= nt; i++) {
        rt_gguf_tensor_info ti;
        if (rt_gguf_tensor_info_at(g, i, &ti) == RT_OK) {
            uint64_t idx = 0;
            (void)rt_gguf_find_tensor(g, ti.name, &idx);
        }
        uint64_t begin = 0, numel = 0;
        std::string why;
        const rt_status rs = rt::gguf_tensor_range(g, size, i, &begin, &numel, why);
        n_ranges++;
        if (rs == RT_OK) {
            // an accepted range lies inside the image: touch its first and last byte
            if (rt_gguf_tensor_info_at(g, i, &ti) == RT_OK && ti.size_in_bytes) {
                volatile uint8_t a = buf[begin], b = buf[begin + ti.size_in_bytes - 1];
                (void)a, (void)b;
            }
        } else n_range_err++;
    }
    rt_gguf_free(g);
    free(buf);
}

static void gguf_cases(const std::vector<uint8_t> &img) {
    walk(img.data(), img.size());
    for (uint64_t cut = 0; cut < img.size(); cut++) walk(img.data(), cut);
    std::vector<uint8_t> m;
    for (int it = 0; it < 3000; it++) {
        m = img;
        const int kind = (int)(rnd() % 4);
        const uint64_t pos = rnd() % m.size();
        if (kind == 0) m[pos] = (uint8_t)rnd();
        else if (kind == 1) m[pos] ^= (uint8_t)(1u << (rnd() % 8));
        else { // an 8-byte field replaced by a hostile value
            static const uint64_t bad[] = {0, 1, 0x7fffffffffffffffull, 0x8000000000000000ull, UINT64_MAX, UINT64_MAX - 7,
                                           UINT64_MAX - 31, 1ull << 32, (1ull << 62) + 5, 0xffffffffull};
            const uint64_t v = bad[rnd() % (sizeof(bad) / sizeof(bad[0]))];
            const uint64_t p8 = pos + 8 <= m.size() ? pos : (m.size() >= 8 ? m.size() - 8 : 0);
            if (m.size() >= 8) memcpy(&m[p8], &v, 8);
        }
        walk(m.data(), m.size());
    }
    // a tensor offset of 2^64 - k (k below the data offset): begin + offset would wrap to a small number
    for (uint64_t pos = 0; pos + 8 <= img.size(); pos++) {
        m = img;
        const uint64_t v = UINT64_MAX - (pos % 64);
        memcpy(&m[pos], &v, 8);
        walk(m.data(), m.size());
    }
}

static long n_desc = 0;
static void matmul_cases() {
    static const int64_t ext[] = {0, 1, 2, 3, 31, 32, 33, 256, 2560, (int64_t)1 << 31, (int64_t)1 << 62, -1};
    const int NE = sizeof(ext) / sizeof(ext[0]);
    for (int it = 0; it < 200000; it++) {
        rt_matmul_desc d;
        memset(&d, 0, sizeof d);
        d.lhs_dt = (int)(rnd() % 8) - 1, d.rhs_dt = (int)(rnd() % 8) - 1;
        d.lhs_rank = (int)(rnd() % 11) - 1, d.rhs_rank = (int)(rnd() % 11) - 1; // -1 .. 9: beyond RT_MAX_RANK too
        for (int i = 0; i < RT_MAX_RANK; i++) d.lhs_shape[i] = ext[rnd() % NE], d.rhs_shape[i] = ext[rnd() % NE];
        if (rnd() % 2) { // make the contraction agree half of the time so that deeper code runs
            const int64_t k = ext[1 + rnd() % 8];
            if (d.lhs_rank >= 1 && d.lhs_rank <= RT_MAX_RANK) d.lhs_shape[d.lhs_rank - 1] = k;
            if (d.rhs_rank >= 1 && d.rhs_rank <= RT_MAX_RANK) d.rhs_shape[d.rhs_rank - 1] = k;
        }
        d.trans_lhs = (int)(rnd() % 2), d.trans_rhs = (int)(rnd() % 2), d.trans_out = (int)(rnd() % 2);
        d.has_bias = (int)(rnd() % 2), d.bias_dt = (int)(rnd() % 8) - 1, d.bias_rank = (int)(rnd() % 4);
        for (int i = 0; i < RT_MAX_RANK; i++) d.bias_shape[i] = ext[rnd() % NE];
        rt::Shape out;
        int out_dt = 0;
        std::string why;
        try { // the C entry points catch what the rules throw; so does this
            (void)rt::validate(d, &why);
            (void)rt::infer(d, out, out_dt, &why);
            rt_gemm_spec spec;
            rt::Problem p;
            (void)rt::make_spec(d, spec, p, &why);
        } catch (const std::exception &) {
        }
        n_desc++;
    }
}

int main(int argc, char **argv) {
    for (int a = 1; a < argc; a++) {
        FILE *f = fopen(argv[a], "rb");
        if (!f) { fprintf(stderr, "cannot open %s\n", argv[a]); return 2; }
        std::vector<uint8_t> img;
        uint8_t chunk[4096];
        size_t n;
        while ((n = fread(chunk, 1, sizeof chunk, f)) > 0) img.insert(img.end(), chunk, chunk + n);
        fclose(f);
        gguf_cases(img);
    }
    matmul_cases();
    printf("ok parsed=%ld rejected=%ld ranges=%ld ranges_rejected=%ld descriptors=%ld\n", n_ok, n_err, n_ranges, n_range_err, n_desc);
    return 0;
}
