// Graph-side host code under AddressSanitizer and UBSan, built and driven by tests/test_host_fold.py: the matchers
// of include/ovfcc_graph.h and the step from a matched node and its Constants' bytes to the arrays
// ovfcc_weights_create takes.  Reads graphs (node arrays plus constant data) from a case file, keeps every Constant
// in a heap block of exactly its size, runs the matcher each case names and the constant handling for every node it
// finds, and writes folds and arrays to an output file for the test to compare.  Every node of every graph is also
// offered to every matcher as a root, results ignored: refusals must be as clean as matches.  No GPU.
//
//   case file:  int32 n_cases, then per case  int32 kind, root, n_nodes; ovfcc_gnode[n_nodes];
//               per node int64 n_bytes (-1: no data) and the bytes
//   kinds:      0 ovfcc_fold_match  1 ovfcc_fold_gather_matmul  2 ovfcc_fold_grouped_matmul  3 ovfcc_fold_moe
//               4 ovfcc_fold_model
//   output:     per case int32 rc, then (rc == 0) the fold structures and one record per created node:
//               int32 rc; ovfcc_fc_desc; int64 n + bytes of weights, scales (f16), zero-points, bias (f16)
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <vector>

#include "ovfcc_graph.h"
#include "ovfcc_internal.h"

#include "launch_stubs.h"

namespace {

FILE* g_out = nullptr;

template <class T>
void put(const T& v) {
    std::fwrite(&v, sizeof(T), 1, g_out);
}
void put_bytes(const void* p, size_t n) {
    put<int64_t>((int64_t)n);
    if (n)
        std::fwrite(p, 1, n, g_out);
}
template <class T>
bool get(FILE* f, T& v) {
    return std::fread(&v, sizeof(T), 1, f) == 1;
}

void record(int rc, const ovfcc::FoldConstants& c) {
    put<int32_t>(rc);
    if (rc)
        return;
    put(c.desc);
    const bool four = c.desc.w_type == OVFCC_U4 || c.desc.w_type == OVFCC_I4;
    const size_t count = (size_t)(c.desc.N * c.desc.K);
    put_bytes(c.weights, four ? (count + 1) / 2 : count);
    put_bytes(c.scales.data(), c.scales.size() * 2);
    put_bytes(c.zero_points.data(), c.zero_points.size());
    put_bytes(c.bias.data(), c.bias.size() * 2);
}

void experts(const std::vector<ovfcc_gnode>& nodes, const ovfcc_gather_fold& f, const void* const* data) {
    for (int e = 0; e < f.n_experts; ++e) {
        ovfcc::FoldConstants c;
        record(ovfcc::fold_expert_constants(nodes.data(), (int)nodes.size(), f, e, data, c), c);
    }
    ovfcc::FoldConstants c;  // one past the end is refused
    if (ovfcc::fold_expert_constants(nodes.data(), (int)nodes.size(), f, f.n_experts, data, c) == OVFCC_OK)
        std::abort();
}

}  // namespace

int main(int argc, char** argv) {
    if (argc != 3)
        return 2;
    FILE* in = std::fopen(argv[1], "rb");
    g_out = std::fopen(argv[2], "wb");
    if (!in || !g_out)
        return 2;
    int32_t n_cases = 0;
    if (!get(in, n_cases))
        return 2;
    for (int32_t ci = 0; ci < n_cases; ++ci) {
        int32_t kind, root, n_nodes;
        if (!get(in, kind) || !get(in, root) || !get(in, n_nodes) || n_nodes <= 0)
            return 3;
        std::vector<ovfcc_gnode> nodes((size_t)n_nodes);
        if (std::fread(nodes.data(), sizeof(ovfcc_gnode), (size_t)n_nodes, in) != (size_t)n_nodes)
            return 3;
        std::vector<std::unique_ptr<uint8_t[]>> blocks((size_t)n_nodes);
        std::vector<const void*> data((size_t)n_nodes, nullptr);
        for (int i = 0; i < n_nodes; ++i) {
            int64_t nb;
            if (!get(in, nb))
                return 3;
            if (nb < 0)
                continue;
            blocks[(size_t)i].reset(new uint8_t[(size_t)nb]);  // exactly sized: an over-read is a sanitizer report
            if (nb && std::fread(blocks[(size_t)i].get(), 1, (size_t)nb, in) != (size_t)nb)
                return 3;
            data[(size_t)i] = blocks[(size_t)i].get();
        }
        const ovfcc_gnode* N = nodes.data();
        if (kind == 0) {
            ovfcc_fold f;
            std::memset(&f, 0, sizeof f);
            const int rc = ovfcc_fold_match(N, n_nodes, root, &f);
            put<int32_t>(rc);
            if (rc == OVFCC_OK) {
                put(f);
                ovfcc::FoldConstants c;
                record(ovfcc::fold_constants(N, n_nodes, f, data.data(), c), c);
            }
        } else if (kind == 1 || kind == 2) {
            ovfcc_gather_fold f;
            std::memset(&f, 0, sizeof f);
            const int rc = kind == 1 ? ovfcc_fold_gather_matmul(N, n_nodes, root, &f) : ovfcc_fold_grouped_matmul(N, n_nodes, root, &f);
            put<int32_t>(rc);
            if (rc == OVFCC_OK) {
                put(f);
                experts(nodes, f, data.data());
            }
        } else if (kind == 3) {
            ovfcc_moe_fold m;
            std::memset(&m, 0, sizeof m);
            const int rc = ovfcc_fold_moe(N, n_nodes, root, &m);
            put<int32_t>(rc);
            if (rc == OVFCC_OK) {
                put(m);
                experts(nodes, m.gate, data.data());
                experts(nodes, m.up, data.data());
                experts(nodes, m.down, data.data());
            }
        } else if (kind == 4) {
            std::vector<ovfcc_fold> folds((size_t)n_nodes + 1);
            std::vector<ovfcc_fused> fused((size_t)n_nodes + 1);
            std::memset(folds.data(), 0, folds.size() * sizeof(ovfcc_fold));
            std::memset(fused.data(), 0, fused.size() * sizeof(ovfcc_fused));
            int nf = 0, nu = 0;
            const int rc = ovfcc_fold_model(N, n_nodes, folds.data(), (int)folds.size(), &nf, fused.data(), (int)fused.size(), &nu);
            put<int32_t>(rc);
            if (rc == OVFCC_OK) {
                put<int32_t>(nf);
                for (int i = 0; i < nf; ++i)
                    put(folds[(size_t)i]);
                put<int32_t>(nu);
                for (int i = 0; i < nu; ++i)
                    put(fused[(size_t)i]);
                for (int i = 0; i < nf; ++i) {
                    ovfcc::FoldConstants c;
                    record(ovfcc::fold_constants(N, n_nodes, folds[(size_t)i], data.data(), c), c);
                }
                // arrays that are too small are refused, not overrun
                int a = 0, b = 0;
                if (nf > 0 && ovfcc_fold_model(N, n_nodes, folds.data(), nf - 1, &a, fused.data(), (int)fused.size(), &b) == OVFCC_OK)
                    std::abort();
            }
        } else {
            return 3;
        }
        // every node as a root of every matcher
        for (int r = -1; r <= n_nodes; ++r) {
            ovfcc_fold f;
            ovfcc_gather_fold gf;
            ovfcc_moe_fold mf;
            (void)ovfcc_fold_match(N, n_nodes, r, &f);
            (void)ovfcc_fold_gather_matmul(N, n_nodes, r, &gf);
            (void)ovfcc_fold_grouped_matmul(N, n_nodes, r, &gf);
            (void)ovfcc_fold_moe(N, n_nodes, r, &mf);
        }
    }
    std::fclose(in);
    std::fclose(g_out);
    std::printf("%d cases\n", n_cases);
    return 0;
}
