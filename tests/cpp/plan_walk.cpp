// Host-only walk over the argument checks of the C ABI: cq_plan_kind (the entry points' own validation and kernel
// choice, without a launch) and the size helpers over every operation x float type x value x parameter type x store
// x block shape x tensor shape x layout, valid and invalid alike, plus damaged descriptors (rank 9, element size 3,
// null pointers).  No pointer is dereferenced by the library and nothing is launched, so it runs without a GPU.
// Exit code 0 and a count of calls per status (2: a call answered CQ_OK without naming a kernel family).  Also meant
// to be built with -fsanitize=address,undefined against a library whose host side is built the same way
// (hipcc: -Xarch_host -fsanitize=address -Xarch_host -fsanitize=undefined).
#include "cubek_quant.h"
#include <cstdio>
#include <cstdint>
#include <vector>
#include <random>
int main() {
    std::mt19937_64 rng(7);
    const std::vector<std::vector<uint64_t>> shapes = {
        {0}, {1}, {7}, {32}, {4096}, {1024, 1024}, {28672, 8192}, {3, 5}, {64, 0}, {2, 3, 128}, {8, 4096, 32, 128},
        {1, 1, 1, 32}, {5, 4104}, {14336, 4096}, {33, 24}, {16, 8184}, {2, 2, 2, 2, 2, 2, 2, 64}, {4294967296ull, 2}};
    const std::vector<std::vector<uint8_t>> blocks = {{}, {32}, {24}, {64}, {128, 128}, {1, 64}, {4, 8, 16}, {1, 1, 1, 1, 32}, {8}, {255}, {0}, {3}};
    uint64_t calls = 0; uint64_t by_status[16] = {0};
    char dummy[64];
    for (int op = 0; op <= 7; op++)
    for (int dtype = 0; dtype <= 3; dtype++)
    for (int value = 0; value <= 10; value++)
    for (int param = 0; param <= 3; param++)
    for (int store = 0; store <= 2; store++)
    for (const auto& blk : blocks)
    for (const auto& shape : shapes) {
        for (int layout = 0; layout < 6; layout++) {
            cq_scheme s{}; s.value = value; s.param = param; s.store = store; s.level = blk.empty() ? 0 : 1; s.mode = 0;
            s.block_rank = blk.size(); for (size_t i = 0; i < blk.size(); i++) s.block[i] = blk[i];
            const uint32_t rank = shape.size();
            std::vector<uint64_t> fstr(rank), vshape = shape, vstr(rank), sshape(rank), sstr(rank);
            uint32_t nq = cq_scheme_num_quants(&s); if (nq == 0) nq = 1;
            if (store == 0) vshape[rank - 1] = shape[rank - 1] / nq; else if (value == 6 || value == 9) vshape[rank - 1] = shape[rank - 1] / 2;
            for (uint32_t d = 0; d < rank; d++) {
                const size_t bi = blk.size() + d >= rank ? blk.size() + d - rank : blk.size();
                const uint64_t b = bi < blk.size() && blk[bi] ? blk[bi] : 1;
                sshape[d] = blk.empty() ? 1 : (shape[d] + b - 1) / b;
            }
            auto contiguous = [&](const std::vector<uint64_t>& sh, std::vector<uint64_t>& st, uint64_t pad) {
                uint64_t acc = 1; for (int d = rank - 1; d >= 0; d--) { st[d] = acc; acc *= sh[d] + (d == (int)rank - 1 ? pad : 0); }
            };
            contiguous(shape, fstr, layout == 1 ? 8 : layout == 4 ? 1 : 0);
            contiguous(vshape, vstr, layout == 2 ? 4 : 0);
            contiguous(sshape, sstr, layout == 3 ? 3 : 0);
            if (layout == 5 && rank >= 2) { std::swap(fstr[rank - 1], fstr[rank - 2]); std::swap(sstr[rank - 1], sstr[rank - 2]); }
            if (layout == 3 && rank >= 1) fstr[0] = 0;
            const uint32_t fsz = dtype == 0 ? 4 : 2, psz = param == 0 ? 4 : 2;
            cq_tensor f{dummy, shape.data(), fstr.data(), rank, fsz};
            cq_tensor v{dummy, vshape.data(), vstr.data(), rank, store == 0 ? 4u : 1u};
            cq_tensor sc{dummy, sshape.data(), sstr.data(), blk.empty() ? 1u : rank, op == 0 ? fsz : psz};
            cq_tensor os{dummy, sshape.data(), sstr.data(), blk.empty() ? 1u : rank, psz};
            if (rng() % 97 == 0) f.rank = 9; if (rng() % 89 == 0) v.elem_size = 3; if (rng() % 83 == 0) sc.shape = nullptr;
            uint32_t family = 99;
            const cq_status st = cq_plan_kind((cq_op)op, rng() % 101 ? &f : nullptr, &v, &sc, &os, rng() % 103 ? &s : nullptr, (cq_dtype)dtype, &family);
            by_status[static_cast<unsigned>(st) < 16u ? st : 15]++; calls++;
            if (st == CQ_OK && family > 8u) { printf("CQ_OK without a family: op %d\n", op); return 2; }
            uint64_t n = 1; for (auto e : shape) n *= e;
            (void)cq_workspace_bytes(&s, n);
            for (uint32_t axis = 0; axis <= rank; axis += (rank ? rank : 1)) (void)cq_reduce_workspace_bytes(&f, axis, (cq_dtype)dtype);
        }
    }
    float lo, hi;
    for (int v = 0; v < 256; v++) { (void)cq_value_range(v, &lo, &hi); (void)cq_value_size_bits(v); }
    for (int st = 0; st < 16; st++) (void)cq_strerror((cq_status)st);
    // entry points with arguments that fail validation before anything is launched
    cq_scheme s{}; s.value = 200;
    uint64_t sh[1] = {32}, stx[1] = {1};
    cq_tensor t{dummy, sh, stx, 1, 4};
    printf("quantize bad scheme -> %d\n", cq_quantize(nullptr, &t, &t, &t, &t, &s, CQ_F32));
    printf("dequantize null -> %d\n", cq_dequantize(nullptr, nullptr, &t, &t, &s, CQ_F32));
    printf("calls %llu:", (unsigned long long)calls);
    for (int i = 0; i < 16; i++) printf(" [%d]=%llu", i, (unsigned long long)by_status[i]);
    printf("\n");
    return 0;
}
