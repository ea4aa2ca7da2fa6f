"""The multiply-and-shift division of the pitched-row kernels (cubek_amd/csrc/cq_magic_div.hpp),
compiled for the host and compared with the machine's division: every divisor up to 70000 and a spread
of larger ones, against dividends around the multiples of the divisor, the ends of the range and random ones."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SOURCE = r"""
#include <cstdio>
#include <cstdint>
#include <initializer_list>
#include "cq_magic_div.hpp"
static uint64_t rng = 88172645463325252ull;
static uint32_t next() { rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17; return static_cast<uint32_t>(rng >> 16); }
static int check(uint32_t d) {
    uint32_t magic, shift;
    cq::magic_of(d, &magic, &shift);
    const uint32_t top = 0x7fffffffu;
    const uint32_t q = top / d;
    uint32_t probes[64];
    int n = 0;
    probes[n++] = 0; probes[n++] = 1; probes[n++] = top; probes[n++] = top - 1;
    const uint32_t ks[] = {1, 2, 3, q / 2, q - 1, q};
    for (uint32_t k : ks) {
        if (k == 0 || k > q) continue;
        const uint64_t m = static_cast<uint64_t>(k) * d;
        if (m - 1 <= top) probes[n++] = static_cast<uint32_t>(m - 1);
        if (m <= top) probes[n++] = static_cast<uint32_t>(m);
        if (m + 1 <= top) probes[n++] = static_cast<uint32_t>(m + 1);
    }
    for (int i = 0; i < 24; i++) probes[n++] = next() & top;
    for (int i = 0; i < n; i++)
        if (cq::magic_div(probes[i], magic, shift) != probes[i] / d) {
            std::printf("n=%u d=%u: %u\n", probes[i], d, cq::magic_div(probes[i], magic, shift));
            return 1;
        }
    return 0;
}
int main() {
    for (uint32_t d = 1; d <= 70000; d++) if (check(d)) return 1;
    for (int i = 0; i < 200000; i++) if (check((next() & 0x7fffffffu) | 1u)) return 1;
    for (uint32_t s = 0; s < 31; s++)
        for (uint32_t d : {(1u << s) - 1, 1u << s, (1u << s) + 1}) if (d >= 1 && check(d)) return 1;
    if (check(0x80000000u)) return 1;
    return 0;
}
"""


def test_magic_division_matches_integer_division(tmp_path):
    src = tmp_path / "magic.cpp"
    src.write_text(SOURCE)
    exe = tmp_path / "magic"
    build = subprocess.run(["g++", "-std=c++17", "-O2", "-Wall", "-Wextra", "-Werror",
                            f"-I{os.path.join(ROOT, 'cubek_amd', 'csrc')}", str(src), "-o", str(exe)],
                           stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert build.returncode == 0, build.stdout
    run = subprocess.run([str(exe)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert run.returncode == 0, run.stdout
