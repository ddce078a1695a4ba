// Host-side shape logic of the GEMV dispatch: how two matmul operand shapes are padded to rank 4 and which
// product class (vector.vector, vector.matrix, matrix.vector, matrix.matrix) they form.  Behaviour follows
// gemmBroadcast / getGemmType of the reference (runtime/source/executor/utils/utils.cpp:293-396), including
// the cases where its padding stops short of rank 4; those are reported to the caller instead of being read
// out of range.
#pragma once

#include <stdint.h>

#include "../../include/pimhip.h"

namespace pimhip
{
// A shape of at most kShapeCap entries held in place: the padding below runs once per operator call on the host, so
// it must not touch the heap.
constexpr int kShapeCap = 8;
struct SmallShape {
    int64_t d[kShapeCap];
    int n = 0;
    int64_t& operator[](int i) { return d[i]; }
    int64_t operator[](int i) const { return d[i]; }
    // `count` copies of `v` in front of entry `pos`; false (nothing changed) if they do not fit
    bool insert(int pos, int64_t v, int count = 1)
    {
        if (n + count > kShapeCap) return false;
        for (int i = n - 1; i >= pos; --i) d[i + count] = d[i];
        for (int i = 0; i < count; ++i) d[pos + i] = v;
        n += count;
        return true;
    }
    void prepend_ones_to(int rank)
    {
        if (n < rank) insert(0, 1, rank - n);
    }
};

// Returns false when the ranks differ by more than 3 (the reference aborts there).
inline bool gemm_broadcast(SmallShape& a, SmallShape& b)
{
    for (;;) {
        const int ra = a.n, rb = b.n;
        if (ra == rb) {
            // utils.cpp:299-310: equal ranks are left-padded with ones up to rank 4.
            a.prepend_ones_to(4);
            b.prepend_ones_to(4);
            return true;
        }
        if (ra < rb) {
            const int gap = rb - ra;
            if (gap == 1) {
                // utils.cpp:313-319: a shared leading dim is kept in front, the 1 goes behind it.
                a.insert(a[0] == b[0] ? 1 : 0, 1);
                continue;
            }
            if (gap == 2) {
                // utils.cpp:320-330: three alternatives, no further padding afterwards.
                if (a[0] == b[0]) {
                    a.insert(1, 1, 2);
                } else if (a[0] == b[1]) {
                    a.insert(1, 1);
                    a.insert(0, 1);
                } else if (ra > 1 && rb > 2 && a[1] == b[2]) {
                    a.insert(0, 1, 2);
                }
                return true;
            }
            return false;  // utils.cpp:331-333
        }
        const int gap = ra - rb;
        if (gap == 1) {
            // utils.cpp:337-343: the second operand becomes a row block (1 in front) when its rows match the
            // first operand's columns, else a column (1 behind).
            if (rb >= 2 && a[ra - 1] == b[rb - 2])
                b.insert(0, 1);
            else
                b.insert(b.n, 1);
            continue;
        }
        if (gap == 2) {
            // utils.cpp:344-355 (reads a[3]: only reachable with ra == 4, rb == 2).
            if (ra == 4 && a[3] == b[1])
                b.insert(b.n, 1);
            else
                b.insert(0, 1);
            b.insert(a[0] == b[0] ? 1 : 0, 1);
            return true;
        }
        if (gap == 3) {
            // utils.cpp:356-366: a rank-1 second operand is laid along the rows if its length equals the
            // first operand's columns, else along the columns; batch dims are copied from the first operand.
            const int64_t len = b[0];
            b = a;
            if (len == a[3]) {
                b[2] = len;
                b[3] = 1;
            } else {
                b[2] = 1;
                b[3] = len;
            }
            return true;
        }
        return false;  // utils.cpp:367-369
    }
}

// utils.cpp:373-396 on two rank-4 shapes.
inline int get_gemm_type(const int64_t* a, const int64_t* b)
{
    if (a[0] != 1 || a[1] != 1 || b[0] != 1 || b[1] != 1) return PIMHIP_GEMM_MM;
    const int na = (a[2] != 1) + (a[3] != 1);
    const int nb = (b[2] != 1) + (b[3] != 1);
    if (na == 1 && nb == 1) return PIMHIP_GEMM_VV;
    if (na == 1 && nb == 2) return PIMHIP_GEMM_VM;
    if (na == 2 && nb == 1) return PIMHIP_GEMM_MV;
    return PIMHIP_GEMM_MM;
}

}  // namespace pimhip
