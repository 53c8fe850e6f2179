// What the C++ tests of the kernel layer share: the check macros and a few accessors written against the public
// interface that DAPHNE's own DenseMatrix has (getValues, getRowSkip, the meta-data object), so that the same test
// code compiles against the stand-in data structures and against the reference's.
#pragma once

#include <runtime/local/datastructures/DataObjectFactory.h>
#include <runtime/local/datastructures/DenseMatrix.h>

#include <cmath>
#include <cstdio>
#include <vector>

static int g_fail = 0, g_checks = 0;
#define CHECK(cond)                                                                                 \
    do {                                                                                            \
        g_checks++;                                                                                 \
        if (!(cond)) {                                                                              \
            g_fail++;                                                                               \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);                           \
        }                                                                                           \
    } while (0)
#define CHECK_THROWS_AS(expr, EX)                                                                   \
    do {                                                                                            \
        g_checks++;                                                                                 \
        bool ok__ = false;                                                                          \
        try {                                                                                       \
            expr;                                                                                   \
        } catch (const EX &) {                                                                      \
            ok__ = true;                                                                            \
        } catch (...) {                                                                             \
        }                                                                                           \
        if (!ok__) {                                                                                \
            g_fail++;                                                                               \
            std::printf("FAILED %s:%d: %s did not throw %s\n", __FILE__, __LINE__, #expr, #EX);     \
        }                                                                                           \
    } while (0)

// the rows x cols values of a matrix (or view) as one contiguous host vector; reads through the const interface,
// so a device-resident matrix is downloaded and both copies stay current
template <class DT> std::vector<typename DT::VT> toHost(const DT *m) {
    const size_t rows = m->getNumRows(), cols = m->getNumCols(), ld = m->getRowSkip();
    std::vector<typename DT::VT> v(rows * cols);
    const typename DT::VT *h = m->getValues();
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < cols; c++)
            v[r * cols + c] = h[r * ld + c];
    return v;
}
// a host matrix with the given values, row by row (genGivenVals of the reference's tests)
template <class DT> DT *given(size_t numRows, const std::vector<typename DT::VT> &vals) {
    const size_t numCols = numRows ? vals.size() / numRows : 0;
    DT *m = DataObjectFactory::create<DT>(numRows, numCols, false);
    typename DT::VT *h = m->getValues();
    for (size_t i = 0; i < vals.size(); i++)
        h[i] = vals[i];
    return m;
}
template <class DT> size_t numDataPlacements(const DT *m) {
    size_t n = 0;
    for (size_t t = 0; t < static_cast<size_t>(ALLOCATION_TYPE::NUM_ALLOC_TYPES); t++)
        n += m->getMetaDataObject()->getDataPlacementByType(static_cast<ALLOCATION_TYPE>(t))->size();
    return n;
}
// bit 0: the host copy is current, bit 1: a device copy is
template <class DT> int whereIs(const DT *m) {
    const MetaDataObject *mdo = m->getMetaDataObject();
    int where = 0;
    for (size_t id : mdo->getLatest())
        where |= mdo->getDataPlacementByID(id)->allocation->getType() == ALLOCATION_TYPE::HOST ? 1 : 2;
    return where;
}

template <class DT> bool equals(const DT *m, const std::vector<typename DT::VT> &exp) { return toHost(m) == exp; }
template <class DT> bool approx(const DT *m, const std::vector<typename DT::VT> &exp, double eps) {
    auto v = toHost(m);
    if (v.size() != exp.size())
        return false;
    for (size_t i = 0; i < v.size(); i++)
        if (!(std::fabs(double(v[i]) - double(exp[i])) <= eps))
            return false;
    return true;
}
