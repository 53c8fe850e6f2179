// C++ host side of the HIP kernel set: the reference's kernel interface on top of the C ABI.
//
// Every kernel is a template struct with a static apply() plus a convenience function, with the
// template parameters, argument order and exception behaviour of the reference's device kernels
// (src/runtime/local/kernels/CUDA/*.h; signatures cited per kernel below), in namespace HIP
// instead of CUDA. `DT *&res`: nullptr on entry makes the kernel allocate the result on the
// device, otherwise it writes in place (res may alias lhs). The last argument is the
// DaphneContext, from which the device context is taken like CUDAContext::get(dctx, deviceID).
//
// This header compiles with a plain host compiler: nothing of HIP leaks through the C ABI. It is
// self-contained so that it can be built and tested without the DAPHNE source tree: DenseMatrix,
// DaphneContext, IContext and DataObjectFactory below are minimal device-resident counterparts
// with the reference's member names (getNumRows / getNumCols / getRowSkip / getValues, ...).
// Inside DAPHNE the same kernel bodies bind to the real classes (getValues(&alloc_desc) for the device pointer).
#pragma once

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include "../../include/daphne_hip.h"

// ------------------------------------------------------------------------------------------
// op codes (src/runtime/local/kernels/BinaryOpCode.h:29-55, UnaryOpCode.h:28-55, AggOpCode.h:25-35)
// ------------------------------------------------------------------------------------------
enum class BinaryOpCode { ADD, SUB, MUL, DIV, POW, MOD, LOG, EQ, NEQ, LT, LE, GT, GE, MIN, MAX, AND, OR, BITWISE_AND, CONCAT };
enum class UnaryOpCode { MINUS, ABS, SIGN, SQRT, EXP, LN, SIN, COS, TAN, ASIN, ACOS, ATAN, SINH, COSH, TANH, FLOOR, CEIL, ROUND, ISNAN, UPPER, LOWER };
enum class AggOpCode { SUM, PROD, MIN, MAX, IDXMIN, IDXMAX, MEAN, STDDEV, VAR };

// ------------------------------------------------------------------------------------------
// contexts (src/runtime/local/context/IContext.h, DaphneContext.h:83-92, CUDAContext.h:29-114)
// ------------------------------------------------------------------------------------------
struct IContext {
    virtual ~IContext() = default;
    virtual void destroy() = 0;
};
struct DaphneContext {
    std::vector<std::unique_ptr<IContext>> hip_contexts; // counterpart of cuda_contexts
    ~DaphneContext() {
        for (auto &c : hip_contexts)
            c->destroy();
    }
    bool useHIP() const { return !hip_contexts.empty(); }
};
#define DCTX(varname) DaphneContext *varname

namespace HIP {
// Re-throws a failed C-ABI status as the exception type the reference throws.
inline void check(dh_status st) {
    if (st == DH_OK)
        return;
    const std::string msg = dh_last_error();
    if (st == DH_ERR_INVALID_ARG)
        throw std::invalid_argument(msg);
    if (st == DH_ERR_DOMAIN)
        throw std::domain_error(msg);
    if (st == DH_ERR_OUT_OF_RANGE)
        throw std::out_of_range(msg);
    throw std::runtime_error(msg);
}
} // namespace HIP

class HIPContext final : public IContext {
    dh_ctx *handle = nullptr;
    int device_id = -1;
    explicit HIPContext(int id) : device_id(id) { HIP::check(dh_ctx_create(id, &handle)); }

  public:
    HIPContext(const HIPContext &) = delete;
    HIPContext &operator=(const HIPContext &) = delete;
    ~HIPContext() override { destroy(); }
    void destroy() override {
        if (handle) {
            dh_ctx_destroy(handle);
            handle = nullptr;
        }
    }
    static std::unique_ptr<IContext> createHipContext(int id) { return std::unique_ptr<IContext>(new HIPContext(id)); }
    static HIPContext *get(DaphneContext *ctx, size_t id) {
        if (ctx == nullptr || id >= ctx->hip_contexts.size())
            throw std::runtime_error("HIPContext::get: no HIP context with this id (createHIPContext not called?)");
        return dynamic_cast<HIPContext *>(ctx->hip_contexts[id].get());
    }
    [[nodiscard]] size_t getMemBudget() const { return dh_ctx_mem_budget(handle); }
    [[nodiscard]] int getDeviceId() const { return device_id; }
    [[nodiscard]] dh_ctx *raw() const { return handle; }
    // CUDAContext::malloc / free: the device pointer is the allocation id
    void *malloc(size_t size, bool zero) {
        void *p = nullptr;
        HIP::check(dh_malloc(handle, size, zero ? 1 : 0, &p));
        return p;
    }
    void free(void *p) { HIP::check(dh_free(handle, p)); }
};

namespace HIP {
// HIP::createHIPContext(DCTX): counterpart of CUDA::createCUDAContext
// (src/runtime/local/kernels/CUDA/CreateCUDAContext.cpp:5-10).
inline void createHIPContext(DCTX(ctx)) { ctx->hip_contexts.emplace_back(HIPContext::createHipContext(0)); }
} // namespace HIP

// ------------------------------------------------------------------------------------------
// device-resident dense matrix (src/runtime/local/datastructures/DenseMatrix.h:42-56,201-249)
// ------------------------------------------------------------------------------------------
template <typename ValueType> class DenseMatrix {
    size_t numRows, numCols, rowSkip;
    ValueType *values;          // device pointer (first element of this view)
    std::shared_ptr<void> buf;  // the allocation; shared by views
    HIPContext *hctx;

  public:
    using VT = ValueType;
    DenseMatrix(size_t rows, size_t cols, bool zero, HIPContext *hc)
        : numRows(rows), numCols(cols), rowSkip(cols), hctx(hc) {
        void *p = hc->malloc(std::max<size_t>(1, rows * cols) * sizeof(VT), zero);
        buf = std::shared_ptr<void>(p, [hc](void *q) { hc->free(q); });
        values = static_cast<VT *>(p);
    }
    // view of rows [rl, ru) and columns [cl, cu) (DenseMatrix::sliceRow / slice)
    DenseMatrix(const DenseMatrix *src, size_t rl, size_t ru, size_t cl, size_t cu)
        : numRows(ru - rl), numCols(cu - cl), rowSkip(src->rowSkip), values(src->values + rl * src->rowSkip + cl),
          buf(src->buf), hctx(src->hctx) {}
    [[nodiscard]] size_t getNumRows() const { return numRows; }
    [[nodiscard]] size_t getNumCols() const { return numCols; }
    [[nodiscard]] size_t getRowSkip() const { return rowSkip; }
    [[nodiscard]] size_t getNumItems() const { return numRows * numCols; }
    [[nodiscard]] const VT *getValues() const { return values; }
    VT *getValues() { return values; }
    [[nodiscard]] HIPContext *context() const { return hctx; }
    DenseMatrix *slice(size_t rl, size_t ru, size_t cl, size_t cu) const { return new DenseMatrix(this, rl, ru, cl, cu); }
    DenseMatrix *sliceRow(size_t rl, size_t ru) const { return slice(rl, ru, 0, numCols); }
    // host <-> device (AllocationDescriptor::transferTo / transferFrom)
    void fromHost(const std::vector<VT> &v) {
        for (size_t r = 0; r < numRows; r++)
            HIP::check(dh_h2d(hctx->raw(), values + r * rowSkip, v.data() + r * numCols, numCols * sizeof(VT)));
    }
    [[nodiscard]] std::vector<VT> toHost() const {
        std::vector<VT> v(numRows * numCols);
        for (size_t r = 0; r < numRows; r++)
            HIP::check(dh_d2h(hctx->raw(), v.data() + r * numCols, values + r * rowSkip, numCols * sizeof(VT)));
        return v;
    }
};

struct DataObjectFactory {
    template <class DT> static DT *create(size_t rows, size_t cols, bool zero, DCTX(ctx)) {
        return new DT(rows, cols, zero, HIPContext::get(ctx, 0));
    }
    template <class DT> static void destroy(const DT *m) { delete m; }
};

// genGivenVals of the reference's tests (src/runtime/local/datagen/GenGivenVals.h:68), device side
template <class DT> DT *genGivenVals(size_t numRows, const std::vector<typename DT::VT> &vals, DCTX(ctx)) {
    auto *m = DataObjectFactory::create<DT>(numRows, numRows ? vals.size() / numRows : 0, false, ctx);
    m->fromHost(vals);
    return m;
}

// ------------------------------------------------------------------------------------------
// kernels
// ------------------------------------------------------------------------------------------
namespace HIP {

namespace detail {
template <typename VT> struct is_f32 : std::is_same<VT, float> {};
inline dh_ctx *raw(DCTX(ctx)) { return HIPContext::get(ctx, 0)->raw(); }
} // namespace detail

// The C ABI is overloaded on the value type here so that the templates below stay one-liners.
#define DH_OVERLOAD2(NAME)                                                                                              \
    template <typename... A> inline dh_status NAME(float, A... a) { return NAME##_f32(a...); }                          \
    template <typename... A> inline dh_status NAME(double, A... a) { return NAME##_f64(a...); }
DH_OVERLOAD2(dh_ew_binary)
DH_OVERLOAD2(dh_ew_binary_sca)
DH_OVERLOAD2(dh_ew_unary)
DH_OVERLOAD2(dh_agg_all)
DH_OVERLOAD2(dh_agg_row)
DH_OVERLOAD2(dh_agg_row_idx)
DH_OVERLOAD2(dh_agg_col)
DH_OVERLOAD2(dh_agg_col_idx)
DH_OVERLOAD2(dh_matmul)
DH_OVERLOAD2(dh_syrk)
DH_OVERLOAD2(dh_solve)
DH_OVERLOAD2(dh_conv2d_forward)
DH_OVERLOAD2(dh_maxpool_forward)
DH_OVERLOAD2(dh_affine_forward)
DH_OVERLOAD2(dh_bias_add)
DH_OVERLOAD2(dh_batchnorm_inference)
DH_OVERLOAD2(dh_softmax)
DH_OVERLOAD2(dh_avgpool_forward)
DH_OVERLOAD2(dh_relu_forward)
DH_OVERLOAD2(dh_fill)
DH_OVERLOAD2(dh_col_bind)
DH_OVERLOAD2(dh_extract_col)
DH_OVERLOAD2(dh_transpose)
DH_OVERLOAD2(dh_gemv)
DH_OVERLOAD2(dh_batchnorm_train_forward)
DH_OVERLOAD2(dh_batchnorm_backward)
DH_OVERLOAD2(dh_maxpool_backward)
DH_OVERLOAD2(dh_avgpool_backward)
DH_OVERLOAD2(dh_conv2d_backward_data)
DH_OVERLOAD2(dh_conv2d_backward_filter)
#undef DH_OVERLOAD2
// integer value types, as far as the reference instantiates its device kernels for them
// (kernels/CUDA/EwBinaryMat.cu:267-270, EwBinaryObjSca.cu:91-94, AggAll.cu:155, AggRow.cu:146, AggCol.cu:89,
// Fill.cu:47,49, ColBind.cu:75, ExtractCol.cu:58); any other combination fails to compile, like a missing
// instantiation fails to link there
#define DH_OVERLOAD_INT(NAME, SUF, T)                                                                                   \
    template <typename... A> inline dh_status NAME(T, A... a) { return NAME##_##SUF(a...); }
DH_OVERLOAD_INT(dh_ew_binary, si64, int64_t)
DH_OVERLOAD_INT(dh_ew_binary, ui64, uint64_t)
DH_OVERLOAD_INT(dh_ew_binary, si32, int32_t)
DH_OVERLOAD_INT(dh_ew_binary, ui32, uint32_t)
DH_OVERLOAD_INT(dh_ew_binary_sca, si64, int64_t)
DH_OVERLOAD_INT(dh_ew_binary_sca, ui64, uint64_t)
DH_OVERLOAD_INT(dh_ew_binary_sca, si32, int32_t)
DH_OVERLOAD_INT(dh_ew_binary_sca, ui32, uint32_t)
DH_OVERLOAD_INT(dh_agg_all, si64, int64_t)
DH_OVERLOAD_INT(dh_agg_row, si64, int64_t)
DH_OVERLOAD_INT(dh_agg_row_idx, si64, int64_t)
DH_OVERLOAD_INT(dh_agg_col, si64, int64_t)
DH_OVERLOAD_INT(dh_agg_col_idx, si64, int64_t)
DH_OVERLOAD_INT(dh_fill, si64, int64_t)
DH_OVERLOAD_INT(dh_fill, ui64, uint64_t)
DH_OVERLOAD_INT(dh_col_bind, si64, int64_t)
DH_OVERLOAD_INT(dh_extract_col, si64, int64_t)
DH_OVERLOAD_INT(dh_transpose, si64, int64_t)
#undef DH_OVERLOAD_INT

// --- EwBinaryMat (kernels/CUDA/EwBinaryMat.h:31-47) ---------------------------------------
template <class DTRes, class DTLhs, class DTRhs> struct EwBinaryMat {
    static void apply(BinaryOpCode opCode, DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, DCTX(ctx)) = delete;
};
template <typename VT> struct EwBinaryMat<DenseMatrix<VT>, DenseMatrix<VT>, DenseMatrix<VT>> {
    static void apply(BinaryOpCode opCode, DenseMatrix<VT> *&res, const DenseMatrix<VT> *lhs, const DenseMatrix<VT> *rhs,
                      DCTX(ctx)) {
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<VT>>(lhs->getNumRows(), lhs->getNumCols(), false, ctx);
        check(dh_ew_binary(VT(), detail::raw(ctx), static_cast<int>(opCode), res->getValues(), res->getRowSkip(),
                           lhs->getValues(), lhs->getNumRows(), lhs->getNumCols(), lhs->getRowSkip(), rhs->getValues(),
                           rhs->getNumRows(), rhs->getNumCols(), rhs->getRowSkip()));
    }
};
template <class DTRes, class DTLhs, class DTRhs>
void ewBinaryMat(BinaryOpCode opCode, DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, DCTX(ctx)) {
    EwBinaryMat<DTRes, DTLhs, DTRhs>::apply(opCode, res, lhs, rhs, ctx);
}

// --- EwBinaryObjSca (kernels/CUDA/EwBinaryObjSca.h:37-60) ---------------------------------
template <class DTRes, class DTLhs, typename VTRhs> struct EwBinaryObjSca {
    static void apply(BinaryOpCode opCode, DTRes *&res, const DTLhs *lhs, VTRhs rhs, DCTX(ctx)) = delete;
};
template <typename VT> struct EwBinaryObjSca<DenseMatrix<VT>, DenseMatrix<VT>, VT> {
    static void apply(BinaryOpCode opCode, DenseMatrix<VT> *&res, const DenseMatrix<VT> *lhs, VT rhs, DCTX(ctx)) {
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<VT>>(lhs->getNumRows(), lhs->getNumCols(), false, ctx);
        check(dh_ew_binary_sca(VT(), detail::raw(ctx), static_cast<int>(opCode), res->getValues(), res->getRowSkip(),
                               lhs->getValues(), lhs->getNumRows(), lhs->getNumCols(), lhs->getRowSkip(), rhs));
    }
};
template <class DTRes, class DTLhs, typename VTRhs>
void ewBinaryObjSca(BinaryOpCode opCode, DTRes *&res, const DTLhs *lhs, VTRhs rhs, DCTX(ctx)) {
    EwBinaryObjSca<DTRes, DTLhs, VTRhs>::apply(opCode, res, lhs, rhs, ctx);
}

// --- EwUnaryMat (kernels/EwUnaryMat.h:35-45; no device version in the reference) ----------
template <class DTRes, class DTArg> struct EwUnaryMat {
    static void apply(UnaryOpCode opCode, DTRes *&res, const DTArg *arg, DCTX(ctx)) = delete;
};
template <typename VT> struct EwUnaryMat<DenseMatrix<VT>, DenseMatrix<VT>> {
    static void apply(UnaryOpCode opCode, DenseMatrix<VT> *&res, const DenseMatrix<VT> *arg, DCTX(ctx)) {
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<VT>>(arg->getNumRows(), arg->getNumCols(), false, ctx);
        check(dh_ew_unary(VT(), detail::raw(ctx), static_cast<int>(opCode), res->getValues(), res->getRowSkip(),
                          arg->getValues(), arg->getNumRows(), arg->getNumCols(), arg->getRowSkip()));
    }
};
template <class DTRes, class DTArg> void ewUnaryMat(UnaryOpCode opCode, DTRes *&res, const DTArg *arg, DCTX(ctx)) {
    EwUnaryMat<DTRes, DTArg>::apply(opCode, res, arg, ctx);
}

// --- AggAll (kernels/CUDA/AggAll.h:28-50) -------------------------------------------------
template <typename VTRes, class DTArg> struct AggAll {
    static VTRes apply(AggOpCode opCode, const DTArg *arg, DCTX(ctx)) = delete;
};
template <typename VT> struct AggAll<VT, DenseMatrix<VT>> {
    static VT apply(AggOpCode opCode, const DenseMatrix<VT> *arg, DCTX(ctx)) {
        VT out{};
        check(dh_agg_all(VT(), detail::raw(ctx), static_cast<int>(opCode), arg->getValues(), arg->getNumRows(),
                         arg->getNumCols(), arg->getRowSkip(), &out));
        return out;
    }
};
template <typename VTRes, class DTArg> VTRes aggAll(AggOpCode opCode, const DTArg *arg, DCTX(ctx)) {
    return AggAll<VTRes, DTArg>::apply(opCode, arg, ctx);
}

// --- AggRow (kernels/CUDA/AggRow.h:30-52; IDXMIN / IDXMAX: kernels/AggRow.h:71-94) --------
template <class DTRes, class DTArg> struct AggRow {
    static void apply(AggOpCode opCode, DTRes *&res, const DTArg *arg, DCTX(ctx)) = delete;
};
template <typename VT> struct AggRow<DenseMatrix<VT>, DenseMatrix<VT>> {
    static void apply(AggOpCode opCode, DenseMatrix<VT> *&res, const DenseMatrix<VT> *arg, DCTX(ctx)) {
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<VT>>(arg->getNumRows(), 1, false, ctx);
        check(dh_agg_row(VT(), detail::raw(ctx), static_cast<int>(opCode), res->getValues(), res->getRowSkip(),
                         arg->getValues(), arg->getNumRows(), arg->getNumCols(), arg->getRowSkip()));
    }
};
// RowIdxMin / RowIdxMax: the op's result type is a matrix of size_t (ir/daphneir/DaphneOps.td:544)
template <typename VT> struct AggRow<DenseMatrix<size_t>, DenseMatrix<VT>> {
    static void apply(AggOpCode opCode, DenseMatrix<size_t> *&res, const DenseMatrix<VT> *arg, DCTX(ctx)) {
        static_assert(sizeof(size_t) == sizeof(uint64_t), "indices are 64 bit");
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<size_t>>(arg->getNumRows(), 1, false, ctx);
        check(dh_agg_row_idx(VT(), detail::raw(ctx), static_cast<int>(opCode), reinterpret_cast<uint64_t *>(res->getValues()),
                             res->getRowSkip(), arg->getValues(), arg->getNumRows(), arg->getNumCols(), arg->getRowSkip()));
    }
};
template <class DTRes, class DTArg> void aggRow(AggOpCode opCode, DTRes *&res, const DTArg *arg, DCTX(ctx)) {
    AggRow<DTRes, DTArg>::apply(opCode, res, arg, ctx);
}

// --- AggCol (kernels/CUDA/AggCol.h:30-52) -------------------------------------------------
template <class DTRes, class DTArg> struct AggCol {
    static void apply(AggOpCode opCode, DTRes *&res, const DTArg *arg, DCTX(ctx)) = delete;
};
template <typename VT> struct AggCol<DenseMatrix<VT>, DenseMatrix<VT>> {
    static void apply(AggOpCode opCode, DenseMatrix<VT> *&res, const DenseMatrix<VT> *arg, DCTX(ctx)) {
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<VT>>(1, arg->getNumCols(), false, ctx);
        check(dh_agg_col(VT(), detail::raw(ctx), static_cast<int>(opCode), res->getValues(), arg->getValues(),
                         arg->getNumRows(), arg->getNumCols(), arg->getRowSkip()));
    }
};
template <typename VT> struct AggCol<DenseMatrix<size_t>, DenseMatrix<VT>> {
    static void apply(AggOpCode opCode, DenseMatrix<size_t> *&res, const DenseMatrix<VT> *arg, DCTX(ctx)) {
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<size_t>>(1, arg->getNumCols(), false, ctx);
        check(dh_agg_col_idx(VT(), detail::raw(ctx), static_cast<int>(opCode), reinterpret_cast<uint64_t *>(res->getValues()),
                             arg->getValues(), arg->getNumRows(), arg->getNumCols(), arg->getRowSkip()));
    }
};
template <class DTRes, class DTArg> void aggCol(AggOpCode opCode, DTRes *&res, const DTArg *arg, DCTX(ctx)) {
    AggCol<DTRes, DTArg>::apply(opCode, res, arg, ctx);
}

// --- MatMul (kernels/CUDA/MatMul.h:31-51) -------------------------------------------------
template <class DTRes, class DTLhs, class DTRhs> struct MatMul {
    static void apply(DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, bool transa, bool transb, DCTX(ctx)) = delete;
};
template <typename T> struct MatMul<DenseMatrix<T>, DenseMatrix<T>, DenseMatrix<T>> {
    static void apply(DenseMatrix<T> *&res, const DenseMatrix<T> *lhs, const DenseMatrix<T> *rhs, bool transa,
                      bool transb, DCTX(ctx)) {
        const size_t nr1 = transa ? lhs->getNumCols() : lhs->getNumRows();
        const size_t nc1 = transa ? lhs->getNumRows() : lhs->getNumCols();
        const size_t nr2 = transb ? rhs->getNumCols() : rhs->getNumRows();
        const size_t nc2 = transb ? rhs->getNumRows() : rhs->getNumCols();
        if (nc1 != nr2) // kernels/MatMul.cpp:256-259, before anything is allocated
            throw std::runtime_error("MatMul - #cols of lhs and #rows of rhs must be the same, but got" +
                                     std::to_string(nc1) + "and" + std::to_string(nr2));
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<T>>(nr1, nc2, false, ctx);
        check(dh_matmul(T(), detail::raw(ctx), res->getValues(), res->getRowSkip(), lhs->getValues(), lhs->getNumRows(),
                        lhs->getNumCols(), lhs->getRowSkip(), rhs->getValues(), rhs->getNumRows(), rhs->getNumCols(),
                        rhs->getRowSkip(), transa ? 1 : 0, transb ? 1 : 0));
    }
};
template <class DTRes, class DTLhs, class DTRhs>
void matMul(DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, bool transa, bool transb, DCTX(ctx)) {
    MatMul<DTRes, DTLhs, DTRhs>::apply(res, lhs, rhs, transa, transb, ctx);
}

// --- Syrk (kernels/Syrk.h:30-40 signature with transLeft; device: kernels/CUDA/Syrk.h:29-46) -
template <class DTRes, class DTArg> struct Syrk {
    static void apply(DTRes *&res, const DTArg *arg, bool transLeft, DCTX(ctx)) = delete;
};
template <typename VT> struct Syrk<DenseMatrix<VT>, DenseMatrix<VT>> {
    static void apply(DenseMatrix<VT> *&res, const DenseMatrix<VT> *arg, bool transLeft, DCTX(ctx)) {
        const size_t n = transLeft ? arg->getNumCols() : arg->getNumRows();
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<VT>>(n, n, false, ctx);
        check(dh_syrk(VT(), detail::raw(ctx), res->getValues(), res->getRowSkip(), arg->getValues(), arg->getNumRows(),
                      arg->getNumCols(), arg->getRowSkip(), transLeft ? 1 : 0));
    }
};
template <class DTRes, class DTArg> void syrk(DTRes *&res, const DTArg *arg, bool transLeft, DCTX(ctx)) {
    Syrk<DTRes, DTArg>::apply(res, arg, transLeft, ctx);
}

// --- Solve (kernels/CUDA/Solve.h; checks of kernels/Solve.h:93-101) ------------------------
template <class DTRes, class DTLhs, class DTRhs> struct Solve {
    static void apply(DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, DCTX(ctx)) = delete;
};
template <typename VT> struct Solve<DenseMatrix<VT>, DenseMatrix<VT>, DenseMatrix<VT>> {
    static void apply(DenseMatrix<VT> *&res, const DenseMatrix<VT> *lhs, const DenseMatrix<VT> *rhs, DCTX(ctx)) {
        if (lhs->getNumRows() != rhs->getNumRows())
            throw std::runtime_error("#rows of lhs and #rows of rhs must be the same");
        if (lhs->getNumRows() != lhs->getNumCols())
            throw std::runtime_error("#rows and #cols of lhs must be the same");
        if (lhs->getRowSkip() != lhs->getNumCols())
            throw std::runtime_error("#cols of lhs must match row skip");
        if (rhs->getNumCols() != 1)
            throw std::runtime_error("#cols of rhs must be 1");
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<VT>>(lhs->getNumRows(), 1, false, ctx);
        check(dh_solve(VT(), detail::raw(ctx), res->getValues(), lhs->getValues(), lhs->getNumRows(), lhs->getRowSkip(),
                       rhs->getValues()));
    }
};
template <class DTRes, class DTLhs, class DTRhs> void solve(DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, DCTX(ctx)) {
    Solve<DTRes, DTLhs, DTRhs>::apply(res, lhs, rhs, ctx);
}

// --- Convolution::Forward (kernels/CUDA/Convolution.h:33-38) -------------------------------
namespace Convolution {
template <class DTRes, class DTArg> struct Forward {
    static void apply(DTRes *&res, size_t *res_h, size_t *res_w, const DTArg *data, const DTArg *filter, const DTArg *bias,
                      const size_t batch_size, const size_t num_channels, const size_t img_h, const size_t img_w,
                      const size_t filter_h, const size_t filter_w, const size_t stride_h, const size_t stride_w,
                      const size_t pad_h, const size_t pad_w, DCTX(ctx)) {
        using VT = typename DTRes::VT;
        const size_t F = filter->getNumRows();
        const size_t P = (img_h + 2 * pad_h - filter_h) / stride_h + 1, Q = (img_w + 2 * pad_w - filter_w) / stride_w + 1;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(batch_size, F * P * Q, false, ctx);
        // the CUDA kernel skips the bias when it is null or aliases the filter (Convolution.cpp:119-121)
        const VT *b = (bias && bias != filter) ? bias->getValues() : nullptr;
        check(dh_conv2d_forward(VT(), detail::raw(ctx), res->getValues(), res_h, res_w, data->getValues(),
                                filter->getValues(), filter->getNumRows(), filter->getNumCols(), b, batch_size,
                                num_channels, img_h, img_w, filter_h, filter_w, stride_h, stride_w, pad_h, pad_w));
    }
};
} // namespace Convolution

// --- NN::Pooling::Forward<MAX | AVG> (kernels/CUDA/Pooling.h:31-35) ------------------------
namespace NN::Pooling {
template <typename VT> struct MAX {};
template <typename VT> struct AVG {};
template <template <typename> class OP, class DTRes, class DTArg> struct Forward {
    static void apply(DTRes *&res, size_t &res_h, size_t &res_w, const DTArg *data, const size_t batch_size,
                      const size_t num_channels, const size_t img_h, const size_t img_w, const size_t pool_h,
                      const size_t pool_w, const size_t stride_h, const size_t stride_w, const size_t pad_h,
                      const size_t pad_w, DCTX(ctx)) {
        using VT = typename DTRes::VT;
        const size_t P = (img_h + 2 * pad_h - pool_h) / stride_w + 1, Q = (img_w + 2 * pad_w - pool_w) / stride_h + 1;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(batch_size, num_channels * P * Q, false, ctx);
        if constexpr (std::is_same<OP<VT>, MAX<VT>>::value)
            check(dh_maxpool_forward(VT(), detail::raw(ctx), res->getValues(), &res_h, &res_w, data->getValues(),
                                     batch_size, num_channels, img_h, img_w, pool_h, pool_w, stride_h, stride_w, pad_h,
                                     pad_w));
        else
            check(dh_avgpool_forward(VT(), detail::raw(ctx), res->getValues(), &res_h, &res_w, data->getValues(),
                                     batch_size, num_channels, img_h, img_w, pool_h, pool_w, stride_h, stride_w, pad_h,
                                     pad_w));
    }
};
} // namespace NN::Pooling

// --- NN::Affine::Forward (kernels/CUDA/Affine.h:24-26) --------------------------------------
namespace NN::Affine {
template <class DTRes, class DTArg> struct Forward {
    static void apply(DTRes *&res, const DTArg *data, const DTArg *weights, const DTArg *bias, DCTX(ctx)) {
        using VT = typename DTRes::VT;
        if (data->getNumCols() != weights->getNumRows())
            throw std::runtime_error("CUDA::NN::Affine: #cols of lhs and #rows of rhs must be the same (" +
                                     std::to_string(data->getNumCols()) + " != " + std::to_string(weights->getNumRows()) + ")");
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(data->getNumRows(), weights->getNumCols(), false, ctx);
        check(dh_affine_forward(VT(), detail::raw(ctx), res->getValues(), data->getValues(), data->getNumRows(),
                                data->getNumCols(), weights->getValues(), weights->getNumRows(), weights->getNumCols(),
                                bias ? bias->getValues() : nullptr, bias ? bias->getNumRows() : 0,
                                bias ? bias->getNumCols() : 0));
    }
};
} // namespace NN::Affine

// --- BiasAdd (kernels/CUDA/BiasAdd.h:26-28) -------------------------------------------------
template <class DTRes, class DTArg> struct BiasAdd {
    static void apply(DTRes *&res, const DTArg *data, const DTArg *bias, DCTX(ctx)) {
        using VT = typename DTRes::VT;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(data->getNumRows(), data->getNumCols(), false, ctx);
        check(dh_bias_add(VT(), detail::raw(ctx), res->getValues(), data->getValues(), data->getNumRows(),
                          data->getNumCols(), bias->getValues(), bias->getNumItems()));
    }
};

// --- BatchNormInferenceForward (kernels/CUDA/BatchNorm.h:26-29) -----------------------------
template <class DTRes, class DTArg> struct BatchNormInferenceForward {
    static void apply(DTRes *&res, const DTArg *data, const DTArg *gamma, const DTArg *beta, const DTArg *ema_mean,
                      const DTArg *ema_var, const typename DTArg::VT eps, DCTX(ctx)) {
        using VT = typename DTRes::VT;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(data->getNumRows(), data->getNumCols(), false, ctx);
        check(dh_batchnorm_inference(VT(), detail::raw(ctx), res->getValues(), data->getValues(), data->getNumRows(),
                                     data->getNumCols(), gamma->getValues(), beta->getValues(), ema_mean->getValues(),
                                     ema_var->getValues(), gamma->getNumRows(), eps, 0));
    }
};

// --- Softmax (kernels/CUDA/Softmax.h:32-34) -------------------------------------------------
template <class DTRes, class DTArg> struct Softmax {
    static void apply(DTRes *&res, const DTArg *data, DCTX(ctx)) {
        using VT = typename DTRes::VT;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(data->getNumRows(), data->getNumCols(), false, ctx);
        check(dh_softmax(VT(), detail::raw(ctx), res->getValues(), res->getRowSkip(), data->getValues(),
                         data->getNumRows(), data->getNumCols(), data->getRowSkip()));
    }
};

// --- NN::Activation::Forward<ReLU> (kernels/CUDA/Activation.h:24-33) -----------------------
namespace NN::Activation {
struct ReLU {};
template <typename OP, typename DTRes, typename DTArg> struct Forward {
    static void apply(DTRes *&res, const DTArg *data, DCTX(ctx)) {
        using VT = typename DTRes::VT;
        static_assert(std::is_same<OP, ReLU>::value, "ReLU is the only activation of the reference's kernel library");
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(data->getNumRows(), data->getNumCols(), false, ctx);
        check(dh_relu_forward(VT(), detail::raw(ctx), res->getValues(), res->getRowSkip(), data->getValues(),
                              data->getNumRows(), data->getNumCols(), data->getRowSkip()));
    }
};
} // namespace NN::Activation

// --- Fill (kernels/CUDA/Fill.h:30-47) --------------------------------------------------------
template <class DTRes, typename VTArg> struct Fill {
    static void apply(DTRes *&res, VTArg arg, size_t numRows, size_t numCols, DCTX(ctx)) {
        using VT = typename DTRes::VT;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(numRows, numCols, false, ctx);
        check(dh_fill(VT(), detail::raw(ctx), res->getValues(), res->getRowSkip(), static_cast<VT>(arg), numRows, numCols));
    }
};
template <class DTRes, typename VTArg> void fill(DTRes *&res, VTArg arg, size_t numRows, size_t numCols, DCTX(ctx)) {
    Fill<DTRes, VTArg>::apply(res, arg, numRows, numCols, ctx);
}

// --- ColBind (kernels/CUDA/ColBind.h:26-44) --------------------------------------------------
template <class DTRes, class DTLhs, class DTRhs> struct ColBind {
    static void apply(DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, DCTX(ctx)) {
        using VT = typename DTRes::VT;
        if (lhs->getNumRows() != rhs->getNumRows())
            throw std::runtime_error("ColBind - the two operands must have the same number of rows, but lhs has " +
                                     std::to_string(lhs->getNumRows()) + " and rhs has " +
                                     std::to_string(rhs->getNumRows()) + " rows");
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(lhs->getNumRows(), lhs->getNumCols() + rhs->getNumCols(), false, ctx);
        check(dh_col_bind(VT(), detail::raw(ctx), res->getValues(), res->getRowSkip(), lhs->getValues(), lhs->getNumRows(),
                          lhs->getNumCols(), lhs->getRowSkip(), rhs->getValues(), rhs->getNumRows(), rhs->getNumCols(),
                          rhs->getRowSkip()));
    }
};
template <class DTRes, class DTLhs, class DTRhs> void colBind(DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, DCTX(ctx)) {
    ColBind<DTRes, DTLhs, DTRhs>::apply(res, lhs, rhs, ctx);
}

// --- ExtractCol (kernels/CUDA/ExtractCol.h:26-45); positions as DenseMatrix<int64_t> -------
template <class DTRes, class DTArg, class DTSel> struct ExtractCol {
    static void apply(DTRes *&res, const DTArg *arg, const DTSel *sel, DCTX(ctx)) {
        using VT = typename DTRes::VT;
        static_assert(std::is_same<typename DTSel::VT, int64_t>::value, "column positions are int64_t");
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(arg->getNumRows(), sel->getNumRows(), false, ctx);
        check(dh_extract_col(VT(), detail::raw(ctx), res->getValues(), res->getRowSkip(), arg->getValues(),
                             arg->getNumRows(), arg->getNumCols(), arg->getRowSkip(), sel->getValues(), sel->getNumRows(),
                             sel->getNumCols(), sel->getRowSkip()));
    }
};
template <class DTRes, class DTArg, class DTSel> void extractCol(DTRes *&res, const DTArg *arg, const DTSel *sel, DCTX(ctx)) {
    ExtractCol<DTRes, DTArg, DTSel>::apply(res, arg, sel, ctx);
}

// --- Transpose (kernels/CUDA/Transpose.h:33-47) ----------------------------------------------
template <class DTRes, class DTArg> struct Transpose {
    static void apply(DTRes *&res, const DTArg *arg, DCTX(ctx)) {
        using VT = typename DTRes::VT;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(arg->getNumCols(), arg->getNumRows(), false, ctx);
        check(dh_transpose(VT(), detail::raw(ctx), res->getValues(), res->getRowSkip(), arg->getValues(),
                           arg->getNumRows(), arg->getNumCols(), arg->getRowSkip()));
    }
};
template <class DTRes, class DTArg> void transpose(DTRes *&res, const DTArg *arg, DCTX(ctx)) {
    Transpose<DTRes, DTArg>::apply(res, arg, ctx);
}

// --- Gemv (kernels/CUDA/Gemv.h:34-48): res = t(mat) * vec ------------------------------------
template <class DTRes, class DTMat, class DTVec> struct Gemv {
    static void apply(DTRes *&res, const DTMat *mat, const DTVec *vec, DCTX(ctx)) {
        using VT = typename DTRes::VT;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(mat->getNumCols(), 1, false, ctx);
        check(dh_gemv(VT(), detail::raw(ctx), res->getValues(), res->getRowSkip(), mat->getValues(), mat->getNumRows(),
                      mat->getNumCols(), mat->getRowSkip(), vec->getValues(), vec->getNumRows(), vec->getRowSkip()));
    }
};
template <class DTRes, class DTMat, class DTVec> void gemv(DTRes *&res, const DTMat *mat, const DTVec *vec, DCTX(ctx)) {
    Gemv<DTRes, DTMat, DTVec>::apply(res, mat, vec, ctx);
}

// --- DNN training kernels: the reference has them on the CPU only; same template parameters and argument order ---
// BatchNorm2DTrainForward (kernels/BatchNorm2DTrainForward.h:38-57). The four statistics results are C x 1 here
// (the reference allocates C x C and fills the first C values).
template <class DTRes, class DTArg> struct BatchNorm2DTrainForward {
    static void apply(DTRes *&res, DTRes *&new_emaMean, DTRes *&new_emaVar, DTRes *&mean, DTRes *&invVar, const DTArg *in,
                      const DTArg *gamma, const DTArg *beta, const DTArg *emaMean, const DTArg *emaVar,
                      const typename DTArg::VT eps, const typename DTArg::VT mu, DCTX(ctx)) {
        using VT = typename DTArg::VT;
        const size_t C = gamma->getNumRows() * gamma->getNumCols();
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(in->getNumRows(), in->getNumCols(), false, ctx);
        for (DTRes **m : {&new_emaMean, &new_emaVar, &mean, &invVar})
            if (*m == nullptr)
                *m = DataObjectFactory::create<DTRes>(C, 1, false, ctx);
        check(dh_batchnorm_train_forward(VT(), detail::raw(ctx), res->getValues(), new_emaMean->getValues(),
                                         new_emaVar->getValues(), mean->getValues(), invVar->getValues(), in->getValues(),
                                         in->getNumRows(), in->getNumCols(), gamma->getValues(), beta->getValues(),
                                         emaMean->getValues(), emaVar->getValues(), C, eps, mu));
    }
};
// BatchNorm2DBackward (kernels/BatchNorm2DBackward.h:38-53)
template <class DTRes, class DTArg> struct BatchNorm2DBackward {
    static void apply(DTRes *&dX, DTRes *&dGamma, DTRes *&dBeta, const DTArg *mean, const DTArg *invVar, const DTArg *in,
                      const DTArg *dout, const DTArg *gamma, const typename DTArg::VT eps, DCTX(ctx)) {
        using VT = typename DTArg::VT;
        const size_t C = gamma->getNumRows() * gamma->getNumCols();
        if (dX == nullptr)
            dX = DataObjectFactory::create<DTRes>(in->getNumRows(), in->getNumCols(), false, ctx);
        if (dGamma == nullptr)
            dGamma = DataObjectFactory::create<DTRes>(C, 1, false, ctx);
        if (dBeta == nullptr)
            dBeta = DataObjectFactory::create<DTRes>(C, 1, false, ctx);
        check(dh_batchnorm_backward(VT(), detail::raw(ctx), dX->getValues(), dGamma->getValues(), dBeta->getValues(),
                                    mean->getValues(), invVar->getValues(), in->getValues(), dout->getValues(), in->getNumRows(),
                                    in->getNumCols(), gamma->getValues(), C, eps));
    }
};
// MaxPoolBackward / AvgPoolBackward (kernels/MaxPoolBackward.h:35-40, AvgPoolBackward.h:35-40)
#define DH_POOL_BACKWARD(NAME, FN)                                                                                      \
    template <class DTRes, class DTArg> struct NAME {                                                                   \
        static void apply(DTRes *&res, const DTArg *input, const DTArg *dOut, const size_t batch_size,                  \
                          const size_t num_channels, const size_t img_h, const size_t img_w, const size_t pool_h,       \
                          const size_t pool_w, const size_t stride_h, const size_t stride_w, const size_t pad_h,        \
                          const size_t pad_w, DCTX(ctx)) {                                                              \
            using VT = typename DTArg::VT;                                                                              \
            if (res == nullptr)                                                                                         \
                res = DataObjectFactory::create<DTRes>(batch_size, num_channels * img_h * img_w, false, ctx);           \
            check(FN(VT(), detail::raw(ctx), res->getValues(), input->getValues(), dOut->getValues(), batch_size,       \
                     num_channels, img_h, img_w, pool_h, pool_w, stride_h, stride_w, pad_h, pad_w));                    \
        }                                                                                                               \
    };
DH_POOL_BACKWARD(MaxPoolBackward, dh_maxpool_backward)
DH_POOL_BACKWARD(AvgPoolBackward, dh_avgpool_backward)
#undef DH_POOL_BACKWARD
// Conv2DBackwardData (kernels/Conv2DBackwardData.h:35-46): `output` is the gradient w.r.t. the convolution's result
template <class DTRes, class DTArg> struct Conv2DBackwardData {
    static void apply(const DTArg *filter, const DTArg *output, const size_t stride_h, const size_t stride_w, const size_t pad_h,
                      const size_t pad_w, const size_t input_batch_size, const size_t input_num_channels, const size_t input_h,
                      const size_t input_w, const size_t filter_num_filters, const size_t filter_num_channels,
                      const size_t filter_h, const size_t filter_w, DTRes *&data, DCTX(ctx)) {
        using VT = typename DTArg::VT;
        (void)filter_num_channels;
        if (data == nullptr)
            data = DataObjectFactory::create<DTRes>(input_batch_size, input_num_channels * input_h * input_w, false, ctx);
        check(dh_conv2d_backward_data(VT(), detail::raw(ctx), data->getValues(), filter->getValues(), output->getValues(),
                                      input_batch_size, input_num_channels, input_h, input_w, filter_num_filters, filter_h,
                                      filter_w, stride_h, stride_w, pad_h, pad_w));
    }
};
// Conv2DBackwardFilter (kernels/Conv2DBackwardFilter.h:35-46)
template <class DTRes, class DTArg> struct Conv2DBackwardFilter {
    static void apply(DTRes *&dFilter, const DTArg *input, const DTArg *output, const size_t stride_h, const size_t stride_w,
                      const size_t pad_h, const size_t pad_w, const size_t input_batch_size, const size_t input_num_channels,
                      const size_t input_h, const size_t input_w, const size_t filter_num_filters,
                      const size_t filter_num_channels, const size_t filter_h, const size_t filter_w, DCTX(ctx)) {
        using VT = typename DTArg::VT;
        if (dFilter == nullptr)
            dFilter = DataObjectFactory::create<DTRes>(filter_num_filters, filter_num_channels * filter_h * filter_w, false, ctx);
        check(dh_conv2d_backward_filter(VT(), detail::raw(ctx), dFilter->getValues(), input->getValues(), output->getValues(),
                                        input_batch_size, input_num_channels, input_h, input_w, filter_num_filters, filter_h,
                                        filter_w, stride_h, stride_w, pad_h, pad_w));
    }
};

} // namespace HIP
