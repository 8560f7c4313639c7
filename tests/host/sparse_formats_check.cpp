// Host check of the sparse operand generators and row orders of the harness
// (tensor-core-fp8_amd/GEMM/include/bm_test_utils.h), the counterparts of the reference's
// GenerateUniformBlockedELLIndex, MakeSparseMatrixRandomUniform, IdentityRowSwizzle and
// SortedRowSwizzle (GEMM/include/bm_test_utils.h:48-128, 197-216 there), and of its Host_sddmm
// (172-194 there).  No GPU involved.
// Exit status 0 = every expectation held; each failure prints its line.
#include <cstdio>
#include <set>
#include <vector>

#include "bm_test_utils.h"
#include "fp8gemm.h"

static int g_failures = 0;
#define EXPECT(cond)                                                           \
    do {                                                                       \
        if (!(cond)) {                                                         \
            std::printf("line %d: expectation failed: %s\n", __LINE__, #cond); \
            ++g_failures;                                                      \
        }                                                                      \
    } while (0)

int main()
{
    std::default_random_engine generator;
    // blocked-ELL: every block row stores `nnz` distinct block columns in rising order
    {
        const int ncol = 37, nnz = 9, nrow = 50;
        std::vector<int> ind((size_t)nrow * nnz, -7);
        GenerateUniformBlockedELLIndex(ncol, nnz, nrow, ind.data(), generator);
        std::vector<int> hits(ncol, 0);
        for (int r = 0; r < nrow; ++r)
            for (int j = 0; j < nnz; ++j) {
                const int c = ind[(size_t)r * nnz + j];
                EXPECT(c >= 0 && c < ncol);
                if (j > 0) EXPECT(c > ind[(size_t)r * nnz + j - 1]);
                if (c >= 0 && c < ncol) ++hits[c];
            }
        int used = 0;
        for (int h : hits) used += h > 0;
        EXPECT(used > ncol * 3 / 4);            // a uniform draw reaches most columns over 50 rows
        // every column kept: the list is 0 .. ncol-1
        std::vector<int> all((size_t)ncol);
        GenerateUniformBlockedELLIndex(ncol, ncol, 1, all.data(), generator);
        for (int j = 0; j < ncol; ++j) EXPECT(all[j] == j);
    }
    // compressed sparse rows: exactly `nonzeros` stored entries, rising distinct columns, padding to a multiple
    for (int padding : {0, 4}) {
        const int rows = 40, cols = 90, nonzeros = 700;
        std::vector<e4m3> val((size_t)nonzeros + rows * 4);
        std::vector<int> off(rows + 1, -1), col(val.size(), -1);
        const int64_t stored = MakeSparseMatrixRandomUniform<e4m3, int>(rows, cols, nonzeros, val.data(), off.data(), col.data(), generator, padding);
        EXPECT(off[0] == 0 && off[rows] == stored);
        int64_t real = 0;
        for (int i = 0; i < rows; ++i) {
            EXPECT(off[i + 1] >= off[i]);
            if (padding > 0) EXPECT((off[i + 1] - off[i]) % padding == 0);
            std::set<int> seen;
            bool in_padding = false;
            for (int e = off[i]; e < off[i + 1]; ++e) {
                EXPECT(col[e] >= 0 && col[e] < cols);
                const float v = (float)val[e];
                EXPECT(v > -1.0001f && v < 1.0001f);
                if (seen.count(col[e])) {
                    // only zero-valued padding repeats a column, and it repeats the row's last real one
                    in_padding = true;
                    EXPECT(padding > 0 && v == 0.0f && col[e] == col[e - 1]);
                } else {
                    EXPECT(!in_padding);
                    if (e > off[i]) EXPECT(col[e] > col[e - 1]);
                    seen.insert(col[e]);
                    ++real;
                }
            }
        }
        EXPECT(real == nonzeros);
        if (padding == 0) EXPECT(stored == nonzeros);
        // refused: more entries than places
        EXPECT((MakeSparseMatrixRandomUniform<e4m3, int>(2, 2, 5, val.data(), off.data(), col.data(), generator, 0)) == -1);
        // row orders
        std::vector<int> ident(rows), sorted(rows), viaabi(rows);
        IdentityRowSwizzle(rows, ident.data());
        SortedRowSwizzle(rows, off.data(), sorted.data());
        fp8gemm_sorted_row_swizzle(rows, off.data(), viaabi.data());
        std::set<int> perm(sorted.begin(), sorted.end());
        EXPECT((int)perm.size() == rows);
        for (int i = 0; i < rows; ++i) {
            EXPECT(ident[i] == i);
            EXPECT(sorted[i] == viaabi[i]);
            if (i > 0) EXPECT(off[sorted[i] + 1] - off[sorted[i]] <= off[sorted[i - 1] + 1] - off[sorted[i - 1]]);
        }
    }
    // Host_sddmm: small whole numbers, so that the running fp32 sum equals the integer dot product
    {
        const int m_vec = 5, vec = 3, k = 40, n = 7;
        std::vector<int> li((size_t)m_vec * vec * k), ri((size_t)n * k);
        std::vector<e4m3> lhs(li.size()), rhs(ri.size());
        for (size_t t = 0; t < li.size(); ++t) lhs[t] = e4m3((float)(li[t] = (int)(t * 7 % 13) - 6));
        for (size_t t = 0; t < ri.size(); ++t) rhs[t] = e4m3((float)(ri[t] = (int)(t * 5 % 11) - 5));
        const std::vector<int> off = {0, 2, 2, 5, 6, 9}, col = {1, 6, 0, 3, 4, 2, 0, 5, 6};
        std::vector<float> out(col.size() * vec, -1.0f);
        Host_sddmm<e4m3, float>(m_vec, k, vec, off.data(), col.data(), lhs.data(), rhs.data(), out.data());
        for (int i = 0; i < m_vec; ++i)
            for (int j = off[i]; j < off[i + 1]; ++j)
                for (int v = 0; v < vec; ++v) {
                    long dot = 0;
                    for (int l = 0; l < k; ++l) dot += (long)li[((size_t)i * vec + v) * k + l] * ri[(size_t)col[j] * k + l];
                    EXPECT(out[(size_t)j * vec + v] == (float)dot);
                }
    }
    if (g_failures == 0) std::printf("all checks passed\n");
    return g_failures == 0 ? 0 : 1;
}
