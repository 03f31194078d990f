// kten_hip.hpp — header-only C++17 host side above the C ABI of libkten_hip.so.
//
// It mirrors the raw-tensor half of kten's backend contract with the reference's member
// names, argument meaning and error behaviour, so a compiled host (the JVM through
// JNI / FFM in a kten deployment, or a C++ program) drives the device the same way:
//
//   HipRawTensor          <- AbstractRawTensor    kten-api/.../tensor/store/AbstractRawTensor.kt:5-247
//                            JVMRawTensor         backend/kten-jvm/.../store/JVMRawTensor.kt
//   HipTensorOperations   <- TensorOperations     kten-api/.../tensor/operations/TensorOperations.kt:9-135
//                            OCLTensorOperations  backend/kten-opencl/.../operations/OCLTensorOperations.kt:72-130
//   shape functions       <- ShapeFunctions.kt    kten-api/.../autograd/utils/ShapeFunctions.kt
//   mayUnexpand           <- Utils.kt:14-41       kten-api/.../autograd/functions/Utils.kt
//
// IllegalArgumentException maps to std::invalid_argument, IllegalStateException and device
// failures to std::runtime_error; both are thrown on the host before anything is launched
// where the reference does so. Raw tensors are held through std::shared_ptr (the role JVM
// references play); reference counting of the stores follows OCLRawTensor.kt:21-48.
#pragma once

#include <algorithm>
#include <climits>
#include <cstdint>
#include <functional>
#include <memory>
#include <numeric>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "kten_hip.h"

namespace kten::hip {

using Shape = std::vector<int>;

inline std::string to_string(const Shape& s) {
    std::ostringstream o;
    o << "[";
    for (size_t i = 0; i < s.size(); i++) o << (i ? ", " : "") << s[i];
    o << "]";
    return o.str();
}

// ---------------------------------------------------------------- status -> exception

inline void check(int status) {
    if (status == KTH_OK) return;
    const std::string msg = kth_last_error();
    if (status == KTH_E_ARGUMENT || status == KTH_E_SHAPE) throw std::invalid_argument(msg);
    if (status == KTH_E_MEMORY) throw std::bad_alloc();
    throw std::runtime_error("kth status " + std::to_string(status) + ": " + msg);
}

// ---------------------------------------------------------------- shape functions

inline int64_t toStoreSize(const Shape& s) {                       // ShapeFunctions.kt:344
    return std::accumulate(s.begin(), s.end(), int64_t{1}, std::multiplies<int64_t>());
}

inline int normalizeAxis(const Shape& s, int axis) {               // ShapeFunctions.kt:41-48
    const int res = axis < 0 ? static_cast<int>(s.size()) + axis : axis;
    if (res < 0 || res >= static_cast<int>(s.size()))
        throw std::invalid_argument("Cannot address axis: " + std::to_string(axis) + " in tensor with dimensions: " +
                                    std::to_string(s.size()));
    return res;
}

inline Shape aggregateOver(const Shape& s, int axis, bool keepDimensions) {   // ShapeFunctions.kt:73-83
    const int a = normalizeAxis(s, axis);
    Shape res = s;
    res[a] = 1;
    if (!keepDimensions && res.size() > 1) res.erase(res.begin() + a);
    return res;
}

inline Shape inferExplicitBroadcastShape(const Shape& from, const Shape& to) {   // ShapeFunctions.kt:187-201
    if (from.size() > to.size())
        throw std::invalid_argument("Tensor with shape: " + to_string(from) + " cannot be broadcasted to shape: " + to_string(to));
    Shape padded(to.size() - from.size(), 1);
    padded.insert(padded.end(), from.begin(), from.end());
    Shape out;
    for (size_t i = 0; i < to.size(); i++) {
        if (padded[i] == to[i] || padded[i] == 1) out.push_back(std::max(padded[i], to[i]));
        else throw std::invalid_argument("Shape " + to_string(from) + " must match " + to_string(to) +
                                         " for every non-singleton dimensions (missing dimensions count as singleton "
                                         "dimension at the beginning of the shapes)");
    }
    return out;
}

inline Shape reshapeShape(const Shape& s, const Shape& to) {       // ShapeFunctions.kt:11-39
    int inferred = -1;
    for (size_t i = 0; i < to.size(); i++) {
        if (to[i] < -1) throw std::invalid_argument("Invalid shape: " + to_string(to));
        if (to[i] == -1) {
            if (inferred >= 0) throw std::invalid_argument("Cannot reshape to " + to_string(to) + ". Only one dimension can be inferred");
            inferred = static_cast<int>(i);
        }
    }
    Shape res = to;
    const int64_t elements = toStoreSize(s);
    if (inferred >= 0) {
        res[inferred] = 1;
        const int64_t known = toStoreSize(res);
        res[inferred] = known ? static_cast<int>(elements / known) : 0;
    }
    if (elements != toStoreSize(res))
        throw std::invalid_argument("Cannot reshape tensor with shape: " + to_string(s) + " to shape: " + to_string(to));
    return res;
}

inline Shape unsqueezeShape(const Shape& s, int axis) {            // ShapeFunctions.kt:61-71
    const int n = static_cast<int>(s.size());
    int a;
    if (axis == n) a = axis;
    else if (axis < 0) a = (axis == -(n + 1)) ? 0 : normalizeAxis(s, axis) + 1;
    else a = normalizeAxis(s, axis);
    Shape res = s;
    res.insert(res.begin() + a, 1);
    return res;
}

/// A Kotlin `first..last` range, both ends inclusive; `All` stands for the reference's `all`
/// (kten-api/.../tensor/Constants.kt:7).
struct IntRange {
    int first, last;
    bool operator==(const IntRange& o) const { return first == o.first && last == o.last; }
};
inline constexpr IntRange All{INT32_MIN, INT32_MAX};

inline std::vector<int> normalizeIndex(const Shape& s, const std::vector<int>& index) {   // ShapeFunctions.kt:217-230
    if (index.size() > s.size()) throw std::invalid_argument("Cannot index tensor with shape: " + to_string(s));
    std::vector<int> out;
    for (size_t d = 0; d < index.size(); d++) {
        const int i = index[d] < 0 ? s[d] + index[d] : index[d];
        if (i < 0 || i >= s[d]) throw std::invalid_argument("Cannot index tensor with shape: " + to_string(s));
        out.push_back(i);
    }
    return out;
}

inline std::vector<IntRange> normalizeIndex(const Shape& s, const std::vector<IntRange>& index) {   // ShapeFunctions.kt:240-259
    bool invalid = index.size() > s.size();
    std::vector<IntRange> out;
    for (size_t d = 0; d < index.size() && d < s.size(); d++) {
        IntRange r = index[d];
        if (r == All) r = IntRange{0, s[d] - 1};
        else if (r.first < 0 || r.last < 0) r = IntRange{r.first < 0 ? s[d] + r.first : r.first, r.last < 0 ? s[d] + r.last : r.last};
        if (r.first < 0 || r.last < 0 || r.first >= s[d] || r.last >= s[d] || r.first > r.last) invalid = true;
        out.push_back(r);
    }
    if (invalid) throw std::invalid_argument("Cannot index tensor with shape: " + to_string(s) + " with the given ranges");
    return out;
}

inline Shape permuteShape(const Shape& s, const std::vector<int>& axes) {                 // ShapeFunctions.kt:106-113
    bool ok = s.size() == axes.size();
    for (size_t d = 0; ok && d < s.size(); d++) ok = std::find(axes.begin(), axes.end(), static_cast<int>(d)) != axes.end();
    if (!ok) throw std::invalid_argument("Tensor with shape: " + to_string(s) + " cannot be permuted by the given axes. All dimensions must be indexed.");
    Shape out;
    for (int a : axes) out.push_back(s[a]);
    return out;
}

inline Shape concatShapes(const std::vector<Shape>& shapes, int axis) {                   // ShapeFunctions.kt:85-104
    bool ok = !shapes.empty();
    for (const Shape& sh : shapes) ok = ok && sh.size() == shapes[0].size();
    if (ok) {
        const int a = normalizeAxis(shapes[0], axis);
        int total = 0;
        for (const Shape& sh : shapes) {
            for (size_t d = 0; d < sh.size(); d++) ok = ok && (static_cast<int>(d) == a || sh[d] == shapes[0][d]);
            total += sh[a];
        }
        if (ok) { Shape res = shapes[0]; res[a] = total; return res; }
    }
    throw std::invalid_argument("Cannot concatenate tensors at axis: " + std::to_string(axis) + " (All tensors must have the same number of "
                                "dimenisons, and have the same size at all dimenions except at the dimension indexed by the axis)");
}

enum class AggregatingOperation { SUM = KTH_SUM, MEAN = KTH_MEAN, MAX = KTH_MAX, MIN = KTH_MIN,
                                  ARG_MAX = KTH_ARG_MAX, ARG_MIN = KTH_ARG_MIN };   // AggregatingOperation.kt:3-5

class HipRawTensor;
using Raw = std::shared_ptr<HipRawTensor>;

// ---------------------------------------------------------------- operations object

class HipTensorOperations {
public:
    explicit HipTensorOperations(int device = 0) {
        check(kth_init(device));
        char name[256];
        uint64_t mem = 0;
        int cus = 0, wave = 0;
        check(kth_device_info(name, sizeof(name), &mem, &cus, &wave));
        platformKey = "HIP - " + std::to_string(device) + " - " + name;
        availableMemory = mem;
        computeUnits = cus;
    }

    std::string platformKey;
    uint64_t availableMemory = 0;
    int computeUnits = 0;

    // TensorOperations.kt:11-20
    Raw createRaw(const Shape& shape, const std::function<float(int)>& init);
    Raw createRaw(const Shape& shape);
    Raw createRawFill(const Shape& shape, float constant);
    Raw zerosLike(const Raw& t);                                    // :24
    void zeroOut(const Raw& t);                                     // :26
    Raw pow(float constant, const Raw& t);                          // :39
    Raw concat(int axis, const std::vector<Raw>& inputs);           // :41

    // TensorOperations.kt:129 batchNorm(axis, momentum, epsilon, training): BatchNormOperation
    // (kten-api/.../tensor/operations/nn/BatchNormOperation.kt:5-41). Absent tensors are null.
    struct BatchNormOutputs { Raw output, currentMean, currentStd; };
    struct BatchNormGrads { Raw gradIn, gradGamma, gradBeta; };
    class BatchNorm {
    public:
        BatchNorm(int axis, float momentum, float epsilon, bool training, HipTensorOperations* ops)
            : axis_(axis), momentum_(momentum), epsilon_(epsilon), training_(training), ops_(ops) {}
        BatchNormOutputs calculateOutput(const Raw& input, const Raw& runningMean, const Raw& runningVar, const Raw& gamma, const Raw& beta);
        BatchNormGrads calculateGrads(const Raw& input, const Raw& runningMean, const Raw& runningVar, const Raw& currentMean,
                                      const Raw& currentStd, const Raw& gamma, const Raw& gradOut,
                                      bool inRequiresGrad, bool gammaRequiresGrad, bool betaRequiresGrad);
    private:
        int axis_; float momentum_, epsilon_; bool training_; HipTensorOperations* ops_;
    };
    BatchNorm batchNorm(int axis, float momentum, float epsilon, bool training) { return BatchNorm(axis, momentum, epsilon, training, this); }
    void release(const Raw& t);                                     // :22
    void incrementRef(const Raw& t);                                // :28
    void markSurviveGC(const Raw& t);                               // :30-33 / OCLTensorOperations.kt:96-98
    void markReleasableInGC(const Raw& t);

    // OCLTensorOperations.kt:72-94: every raw tensor constructed while the scope is open is
    // released when it closes; tensors still referenced survive into the next scope.
    class GarbageCollector {
    public:
        explicit GarbageCollector(HipTensorOperations& ops) : ops_(ops), owner_(!ops.collecting_) {
            if (owner_) { ops_.instances_ = ops_.survivors_; ops_.collecting_ = true; }
        }
        ~GarbageCollector() { close(); }
        void close();
    private:
        HipTensorOperations& ops_;
        bool owner_;
        bool closed_ = false;
    };
    GarbageCollector garbageCollector() { return GarbageCollector(*this); }

    void sync() { check(kth_sync()); }

    // Settings of the platform, as the Kotlin module would hold them as platform properties: the tolerance of eq / neq
    // (JVMRawTensor.kt:375-377), the share of device memory the store pool may hold, and how the transcendental maps are
    // evaluated (exact: the float kotlin.math returns, bit for bit; within two ulp: fp32 routines, the default).
    enum class MathMode { EXACT = KTH_MATH_EXACT, WITHIN_2_ULP = KTH_MATH_WITHIN_2_ULP };
    void setEpsilon(float eps) { check(kth_set_epsilon(eps)); }
    void setMemoryUsageScaleHint(double fraction) { check(kth_set_memory_scale_hint(fraction)); }
    void setMathMode(MathMode mode) { check(kth_set_math_mode(static_cast<int>(mode))); }
    MathMode getMathMode() { int m = 0; check(kth_get_math_mode(&m)); return static_cast<MathMode>(m); }

private:
    friend class HipRawTensor;
    void collect(const Raw& t) { if (collecting_) instances_.push_back(t); }
    bool collecting_ = false;
    std::vector<Raw> instances_, survivors_;
};

// ---------------------------------------------------------------- raw tensor

class HipRawTensor : public std::enable_shared_from_this<HipRawTensor> {
public:
    Shape shape;
    uint64_t storeReference;
    HipTensorOperations* ops;
    bool mustSurviveGC = false;

    static Raw make(const Shape& shape, uint64_t handle, HipTensorOperations* ops) {
        Raw t(new HipRawTensor(shape, handle, ops));
        ops->collect(t);
        return t;
    }
    ~HipRawTensor() { if (refCount_ > 0) kth_release(storeReference); }   // safety net

    int dimensions() const { return static_cast<int>(shape.size()); }
    int64_t size() const { return toStoreSize(shape); }

    // --- lifetime (OCLRawTensor.kt:21-48)
    void incrementRef() {
        if (refCount_ <= 0) throw std::runtime_error("Store reference is already released. (Tensor shape: " + to_string(shape) + ")");
        refCount_++;
    }
    bool referenced() const { return refCount_ > 0; }
    bool release() {
        if (refCount_ <= 0) return false;
        if (!mustSurviveGC) refCount_--;
        if (refCount_ == 0) { check(kth_release(storeReference)); return true; }
        return false;
    }

    // --- broadcasting (AbstractRawTensor.kt:25,170-192; JVMRawTensor.kt:51-73)
    Raw broadcastTo(const Shape& to) {
        if (shape == to) return shared_from_this();
        live();
        inferExplicitBroadcastShape(shape, to);
        Raw res = ops->createRaw(to);
        check(kth_broadcast_to(storeReference, shape.data(), dimensions(), res->storeReference, to.data(), static_cast<int>(to.size())));
        return res;
    }
    Shape calculateCommonShapeWith(const HipRawTensor& other) const {
        if (shape == other.shape) return shape;
        Shape a = shape, b = other.shape, res;
        const int diff = static_cast<int>(a.size()) - static_cast<int>(b.size());
        if (diff > 0) { res.assign(a.begin(), a.begin() + diff); a.erase(a.begin(), a.begin() + diff); }
        else if (diff < 0) { res.assign(b.begin(), b.begin() - diff); b.erase(b.begin(), b.begin() - diff); }
        for (size_t i = 0; i < a.size(); i++) res.push_back(std::max(a[i], b[i]));
        return res;
    }

    // --- arithmetic (AbstractRawTensor.kt:39-73)
    Raw plus(const Raw& o) { return binary(KTH_PLUS, o); }
    Raw plus(float c) { return scalar(KTH_PLUS, c); }
    void plusAssign(const Raw& o) { binaryAssign(KTH_PLUS, o); }
    void plusAssign(float c) { scalarAssign(KTH_PLUS, c); }
    Raw minus(const Raw& o) { return binary(KTH_MINUS, o); }
    Raw minus(float c) { return scalar(KTH_MINUS, c); }
    Raw unaryMinus() { return unary(KTH_NEG); }
    Raw times(const Raw& o) { return binary(KTH_TIMES, o); }
    Raw times(float c) { return scalar(KTH_TIMES, c); }
    void timesAssign(const Raw& o) { binaryAssign(KTH_TIMES, o); }
    void timesAssign(float c) { scalarAssign(KTH_TIMES, c); }
    Raw div(const Raw& o) { return binary(KTH_DIV, o); }
    Raw div(float c) { return scalar(KTH_DIV, c); }
    void divAssign(float c) { scalarAssign(KTH_DIV, c); }
    Raw pow(const Raw& o) { return binary(KTH_POW, o); }
    Raw pow(float c) { return scalar(KTH_POW, c); }
    Raw reciprocal() { return unary(KTH_RECIPROCAL); }
    Raw log() { return unary(KTH_LOG); }

    // --- comparisons (AbstractRawTensor.kt:194-206; store-to-store, no broadcast, as on the JVM)
    Raw lt(const Raw& o) { return compare(KTH_LT, o); }    Raw lt(float c) { return scalar(KTH_LT, c); }
    Raw lte(const Raw& o) { return compare(KTH_LTE, o); }  Raw lte(float c) { return scalar(KTH_LTE, c); }
    Raw gt(const Raw& o) { return compare(KTH_GT, o); }    Raw gt(float c) { return scalar(KTH_GT, c); }
    Raw gte(const Raw& o) { return compare(KTH_GTE, o); }  Raw gte(float c) { return scalar(KTH_GTE, c); }
    Raw eq(const Raw& o) { return compare(KTH_EQ, o); }    Raw eq(float c) { return scalar(KTH_EQ, c); }
    Raw neq(const Raw& o) { return compare(KTH_NEQ, o); }  Raw neq(float c) { return scalar(KTH_NEQ, c); }

    // --- pointwise maths (AbstractRawTensor.kt:208-227)
    Raw exp() { return unary(KTH_EXP); }     Raw tanh() { return unary(KTH_TANH); }   Raw sigmoid() { return unary(KTH_SIGMOID); }
    Raw sinh() { return unary(KTH_SINH); }   Raw cosh() { return unary(KTH_COSH); }   Raw abs() { return unary(KTH_ABS); }
    Raw sign() { return unary(KTH_SIGN); }   Raw sqrt() { return unary(KTH_SQRT); }   Raw sin() { return unary(KTH_SIN); }
    Raw cos() { return unary(KTH_COS); }     Raw tan() { return unary(KTH_TAN); }     Raw asin() { return unary(KTH_ASIN); }
    Raw acos() { return unary(KTH_ACOS); }   Raw atan() { return unary(KTH_ATAN); }   Raw floor() { return unary(KTH_FLOOR); }
    Raw ceil() { return unary(KTH_CEIL); }   Raw round() { return unary(KTH_ROUND); } Raw trunc() { return unary(KTH_TRUNC); }
    Raw rsqrt() { return unary(KTH_RSQRT); }
    Raw clamp(float min, float max) {
        live();
        Raw res = ops->createRaw(shape);
        check(kth_clamp(storeReference, res->storeReference, static_cast<uint64_t>(size()), min, max));
        return res;
    }

    // --- reductions (AbstractRawTensor.kt:92-122)
    Raw sum(int axis, bool keepDimensions = false) { return aggregatingOpOverAxis(axis, keepDimensions, AggregatingOperation::SUM); }
    Raw mean(int axis, bool keepDimensions = false) { return aggregatingOpOverAxis(axis, keepDimensions, AggregatingOperation::MEAN); }
    Raw max(int axis, bool keepDimensions = false) { return aggregatingOpOverAxis(axis, keepDimensions, AggregatingOperation::MAX); }
    Raw min(int axis, bool keepDimensions = false) { return aggregatingOpOverAxis(axis, keepDimensions, AggregatingOperation::MIN); }
    Raw argMax(int axis = 0, bool keepDimensions = false) { return aggregatingOpOverAxis(axis, keepDimensions, AggregatingOperation::ARG_MAX); }
    Raw argMin(int axis = 0, bool keepDimensions = false) { return aggregatingOpOverAxis(axis, keepDimensions, AggregatingOperation::ARG_MIN); }
    Raw sum() { return reduceAll(KTH_SUM); }
    Raw mean() { return reduceAll(KTH_MEAN); }

    // --- gather / scatter (AbstractRawTensor.kt:146-164)
    Raw gather(int axis, const Raw& index) {
        live(); index->live();
        const int a = normalizeAxis(shape, axis);
        if (index->dimensions() != dimensions()) throw std::invalid_argument("Gather expects an index with the tensor's dimensions");
        Raw res = ops->createRaw(index->shape);
        check(kth_gather(storeReference, shape.data(), index->storeReference, index->shape.data(), dimensions(), a, res->storeReference));
        return res;
    }
    void inplaceScatter(int axis, const Raw& index, const Raw& src) { scatterImpl(axis, index, src, false); }
    void inplaceScatterAdd(int axis, const Raw& index, const Raw& src) { scatterImpl(axis, index, src, true); }
    void inplaceScatter(int axis, const Raw& index, float src) {
        live(); index->live();
        const int a = normalizeAxis(shape, axis);
        if (index->dimensions() != dimensions()) throw std::invalid_argument("Scatter expects an index with the tensor's dimensions");
        check(kth_scatter_fill(storeReference, shape.data(), index->storeReference, index->shape.data(), dimensions(), a, src));
    }
    Raw scatter(int axis, const Raw& index, const Raw& src) { Raw res = copy(); res->inplaceScatter(axis, index, src); return res; }

    // --- get / set by index and by ranges (AbstractRawTensor.kt:27-37; JVMRawTensor.kt:270-315)
    Raw get(const std::vector<int>& index) {
        live();
        const std::vector<int> norm = normalizeIndex(shape, index);
        int64_t offset, length;
        storeRange(norm, offset, length);
        Raw res = ops->createRaw(norm.size() == shape.size() ? Shape{1} : Shape(shape.begin() + norm.size(), shape.end()));
        check(kth_copy(res->storeReference, 0, storeReference, static_cast<uint64_t>(offset), static_cast<uint64_t>(length)));
        return res;
    }
    Raw get(const std::vector<IntRange>& index) {
        live();
        Shape first, last, resShape;
        fullRanges(normalizeIndex(shape, index), first, last, resShape);
        Raw res = ops->createRaw(resShape);
        check(kth_get_range(storeReference, shape.data(), dimensions(), first.data(), last.data(), res->storeReference));
        return res;
    }
    void set(const std::vector<int>& index, const Raw& value) {
        live(); value->live();
        int64_t offset, length;
        storeRange(normalizeIndex(shape, index), offset, length);
        if (value->size() != length)
            throw std::invalid_argument("Cannot set tensor with shape: " + to_string(value->shape) + " to tensor with shape: " + to_string(shape));
        check(kth_copy(storeReference, static_cast<uint64_t>(offset), value->storeReference, 0, static_cast<uint64_t>(length)));
    }
    void set(const std::vector<int>& index, float value) {
        live();
        int64_t offset, length;
        storeRange(normalizeIndex(shape, index), offset, length);
        check(kth_fill(storeReference, static_cast<uint64_t>(offset), static_cast<uint64_t>(length), value));
    }
    void set(const std::vector<IntRange>& index, const Raw& value) {
        live(); value->live();
        Shape first, last, resShape;
        fullRanges(normalizeIndex(shape, index), first, last, resShape);
        check(kth_set_range(storeReference, shape.data(), dimensions(), first.data(), last.data(), value->storeReference,
                            static_cast<uint64_t>(value->size())));
    }
    void set(const std::vector<IntRange>& index, float value) {
        live();
        Shape first, last, resShape;
        fullRanges(normalizeIndex(shape, index), first, last, resShape);
        check(kth_fill_range(storeReference, shape.data(), dimensions(), first.data(), last.data(), value));
    }

    // --- transpose / permute / narrow / maskedFill (AbstractRawTensor.kt:228-232,246)
    Raw transpose(int axis1, int axis2) {
        live();
        const int a1 = normalizeAxis(shape, axis1), a2 = normalizeAxis(shape, axis2);
        if (a1 == a2) throw std::invalid_argument("Transpose requires different axes as parameters");
        Shape res = shape;
        std::swap(res[a1], res[a2]);
        Raw out = ops->createRaw(res);
        check(kth_transpose(storeReference, shape.data(), dimensions(), a1, a2, out->storeReference));
        return out;
    }
    Raw permute(const std::vector<int>& axes) {
        live();
        Raw out = ops->createRaw(permuteShape(shape, axes));
        check(kth_permute(storeReference, shape.data(), dimensions(), axes.data(), out->storeReference));
        return out;
    }
    Raw narrow(int axis, int start, int length) {                    // JVMRawTensor.kt:468-473
        const int a = normalizeAxis(shape, axis);
        std::vector<IntRange> ranges;
        for (int d : shape) ranges.push_back(IntRange{0, d - 1});
        ranges[a] = IntRange{start, start + length - 1};
        return get(ranges);
    }
    Raw maskedFill(const Raw& mask, float value) {                   // JVMRawTensor.kt:537-540
        live(); mask->live();
        if (mask->shape != shape) inferExplicitBroadcastShape(mask->shape, shape);
        Raw out = ops->createRaw(shape);
        check(kth_masked_fill(storeReference, shape.data(), dimensions(), mask->storeReference, mask->shape.data(),
                              mask->dimensions(), value, out->storeReference));
        return out;
    }

    // --- shape-only members and copies (AbstractRawTensor.kt:77-90,124-144,168)
    Raw copy(bool shallow = false) {
        live();
        if (shallow) { check(kth_retain(storeReference)); return make(shape, storeReference, ops); }
        Raw res = ops->createRaw(shape);
        check(kth_copy(res->storeReference, 0, storeReference, 0, static_cast<uint64_t>(size())));
        return res;
    }
    Raw view(const Shape& to) {
        live();
        Shape s = reshapeShape(shape, to);
        check(kth_retain(storeReference));
        return make(s, storeReference, ops);
    }
    Raw reshape(const Shape& to) { Shape s = reshapeShape(shape, to); Raw res = copy(); res->shape = s; return res; }
    void inplaceReshape(const Shape& to) { shape = reshapeShape(shape, to); }
    void inplaceSqueeze(int axis) { shape.erase(shape.begin() + normalizeAxis(shape, axis)); }
    Raw squeeze(int axis) { Raw res = copy(); res->inplaceSqueeze(axis); return res; }
    void inplaceUnsqueeze(int axis) { shape = unsqueezeShape(shape, axis); }
    Raw unsqueeze(int axis) { Raw res = copy(); res->inplaceUnsqueeze(axis); return res; }

    // --- element access and housekeeping (AbstractRawTensor.kt:166,240,244)
    float getSingleValue(const std::vector<int>& indexes) {
        live();
        if (indexes.size() != shape.size()) throw std::invalid_argument("Cannot index tensor with shape: " + to_string(shape));
        int64_t off = 0;
        for (size_t d = 0; d < shape.size(); d++) {
            const int i = indexes[d] < 0 ? shape[d] + indexes[d] : indexes[d];
            if (i < 0 || i >= shape[d]) throw std::invalid_argument("Cannot index tensor with shape: " + to_string(shape));
            off = off * shape[d] + i;
        }
        float v = 0.0f;
        check(kth_read_scalar(storeReference, static_cast<uint64_t>(off), &v));
        return v;
    }
    bool containsNan() { live(); int flag = 0; check(kth_contains_nan(storeReference, static_cast<uint64_t>(size()), &flag)); return flag != 0; }
    void inplaceFill(float value) { live(); check(kth_fill(storeReference, 0, static_cast<uint64_t>(size()), value)); }
    // inplaceResize (AbstractRawTensor.kt:242; JVMRawTensor.kt:524-531): a new store that keeps the
    // leading values and holds zeros beyond them; this wrapper's reference on the old store is returned.
    void inplaceResize(const Shape& to) {
        live();
        const uint64_t nNew = static_cast<uint64_t>(toStoreSize(to)), nOld = static_cast<uint64_t>(size());
        uint64_t fresh = 0;
        check(kth_alloc(nNew, &fresh));
        const uint64_t kept = nNew < nOld ? nNew : nOld;
        check(kth_copy(fresh, 0, storeReference, 0, kept));
        if (nNew > kept) check(kth_fill(fresh, kept, nNew - kept, 0.0f));
        check(kth_release(storeReference));
        storeReference = fresh;
        shape = to;
    }
    std::vector<float> toVector() {
        live();
        std::vector<float> host(static_cast<size_t>(size()));
        check(kth_download(host.data(), storeReference, 0, host.size()));
        return host;
    }

private:
    HipRawTensor(const Shape& s, uint64_t handle, HipTensorOperations* o) : shape(s), storeReference(handle), ops(o) {}
    int refCount_ = 1;

    void storeRange(const std::vector<int>& norm, int64_t& offset, int64_t& length) const {   // AbstractIndexing.kt:43-54
        int64_t start = 0;
        for (size_t d = 0; d < norm.size(); d++) start = start * shape[d] + norm[d];
        length = 1;
        for (size_t d = norm.size(); d < shape.size(); d++) length *= shape[d];
        offset = start * length;
    }
    void fullRanges(const std::vector<IntRange>& norm, Shape& first, Shape& last, Shape& resShape) const {
        for (size_t d = 0; d < shape.size(); d++) {
            const IntRange r = d < norm.size() ? norm[d] : IntRange{0, shape[d] - 1};
            first.push_back(r.first); last.push_back(r.last);
            resShape.push_back(r.last - r.first + 1);
        }
    }

    void live() const { if (refCount_ <= 0) throw std::runtime_error("Raw tensor with shape " + to_string(shape) + " was released"); }

    Raw binary(int op, const Raw& o) {                              // JVMRawTensor.kt:81-87
        live(); o->live();
        const Shape common = calculateCommonShapeWith(*o);
        if (shape != common) inferExplicitBroadcastShape(shape, common);
        if (o->shape != common) inferExplicitBroadcastShape(o->shape, common);
        Raw res = ops->createRaw(common);
        check(kth_binary(op, storeReference, shape.data(), dimensions(), o->storeReference, o->shape.data(), o->dimensions(),
                         res->storeReference, common.data(), static_cast<int>(common.size())));
        return res;
    }
    void binaryAssign(int op, const Raw& o) {                       // JVMRawTensor.kt:89-97
        live(); o->live();
        if (shape != o->shape)
            throw std::invalid_argument("Shapes does not match for inplace operation on tensors with shapes: " + to_string(shape) +
                                        " and " + to_string(o->shape) + ".");
        check(kth_binary_inplace(op, storeReference, o->storeReference, static_cast<uint64_t>(size())));
    }
    Raw scalar(int op, float c, bool reverse = false) {             // JVMRawTensor.kt:99-103
        live();
        Raw res = ops->createRaw(shape);
        check(kth_scalar(op, storeReference, c, reverse ? 1 : 0, res->storeReference, static_cast<uint64_t>(size())));
        return res;
    }
    void scalarAssign(int op, float c) {                            // JVMRawTensor.kt:105-108
        live();
        check(kth_scalar(op, storeReference, c, 0, storeReference, static_cast<uint64_t>(size())));
    }
    Raw compare(int op, const Raw& o) {
        live(); o->live();
        if (size() != o->size()) throw std::invalid_argument("Comparison needs equally sized tensors");
        Raw res = ops->createRaw(shape);
        const int32_t n = static_cast<int32_t>(size());
        check(kth_binary(op, storeReference, &n, 1, o->storeReference, &n, 1, res->storeReference, &n, 1));
        return res;
    }
    Raw unary(int op) {
        live();
        Raw res = ops->createRaw(shape);
        check(kth_unary(op, storeReference, res->storeReference, static_cast<uint64_t>(size())));
        return res;
    }
    Raw aggregateOverAxis(int axis, const Shape& resShape, AggregatingOperation op) {   // JVMRawTensor.kt:211-225
        live();
        int64_t outer = 1, inner = 1;
        for (int d = 0; d < axis; d++) outer *= shape[d];
        for (int d = axis + 1; d < dimensions(); d++) inner *= shape[d];
        Raw res = ops->createRaw(resShape);
        check(kth_reduce_axis(static_cast<int>(op), storeReference, res->storeReference, static_cast<uint64_t>(outer),
                              static_cast<uint64_t>(shape[axis]), static_cast<uint64_t>(inner)));
        return res;
    }
    Raw aggregatingOpOverAxis(int axis, bool keepDims, AggregatingOperation op) {       // AbstractRawTensor.kt:92-108
        const int a = normalizeAxis(shape, axis);
        const Shape resShape = aggregateOver(shape, a, true);
        Raw res = aggregateOverAxis(a, resShape, op);
        if (!keepDims && resShape.size() > 1) res->shape.erase(res->shape.begin() + a);
        return res;
    }
    Raw reduceAll(int op) {                                         // JVMRawTensor.kt:146-152
        live();
        Raw res = ops->createRaw(Shape{1});
        check(kth_reduce_all(op, storeReference, static_cast<uint64_t>(size()), res->storeReference));
        return res;
    }
    void scatterImpl(int axis, const Raw& index, const Raw& src, bool add) {            // JVMRawTensor.kt:227-255
        live(); index->live(); src->live();
        if (index->dimensions() != dimensions() || src->dimensions() != dimensions())
            throw std::invalid_argument("Scatter expects tensors (target, index, source) to have the same dimensions");
        const int a = normalizeAxis(shape, axis);
        check(kth_scatter(add ? 1 : 0, storeReference, shape.data(), index->storeReference, index->shape.data(),
                          src->storeReference, src->shape.data(), dimensions(), a));
    }
    friend class HipTensorOperations;
};

// ---------------------------------------------------------------- operations: definitions

inline Raw HipTensorOperations::createRaw(const Shape& shape) {
    uint64_t handle = 0;
    check(kth_alloc(static_cast<uint64_t>(toStoreSize(shape)), &handle));
    return HipRawTensor::make(shape, handle, this);
}
inline Raw HipTensorOperations::createRaw(const Shape& shape, const std::function<float(int)>& init) {
    Raw t = createRaw(shape);
    std::vector<float> host(static_cast<size_t>(toStoreSize(shape)));
    for (size_t i = 0; i < host.size(); i++) host[i] = init(static_cast<int>(i));
    check(kth_upload(t->storeReference, 0, host.data(), host.size()));
    return t;
}
inline Raw HipTensorOperations::createRawFill(const Shape& shape, float constant) {
    Raw t = createRaw(shape);
    t->inplaceFill(constant);
    return t;
}
inline Raw HipTensorOperations::zerosLike(const Raw& t) { return createRawFill(t->shape, 0.0f); }
inline void HipTensorOperations::zeroOut(const Raw& t) { t->inplaceFill(0.0f); }
inline Raw HipTensorOperations::pow(float constant, const Raw& t) { return t->scalar(KTH_POW, constant, true); }
inline Raw HipTensorOperations::concat(int axis, const std::vector<Raw>& inputs) {   // TensorOperations.kt:41
    std::vector<Shape> shapes;
    for (const Raw& t : inputs) shapes.push_back(t->shape);
    const Shape resShape = concatShapes(shapes, axis);
    const int a = normalizeAxis(shapes[0], axis);
    Raw res = createRaw(resShape);
    bool anyEmpty = false;
    for (const Raw& t : inputs) anyEmpty = anyEmpty || t->size() == 0;
    if (anyEmpty) {
        // the reference's construction (AbstractJVMTensorOperations.kt:106-120): an empty input is an empty range, which
        // the range set rejects as the reference does
        std::vector<IntRange> target;
        for (int d : resShape) target.push_back(IntRange{0, d - 1});
        int last = 0;
        for (const Raw& t : inputs) {
            target[a] = IntRange{last, last + t->shape[a] - 1};
            res->set(target, t);
            last += t->shape[a];
        }
        return res;
    }
    std::vector<uint64_t> handles;
    std::vector<int32_t> lens;
    for (const Raw& t : inputs) { handles.push_back(t->storeReference); lens.push_back(t->shape[a]); }
    check(kth_concat(handles.data(), lens.data(), static_cast<int>(inputs.size()), resShape.data(), static_cast<int>(resShape.size()), a,
                     res->storeReference));
    return res;
}
inline HipTensorOperations::BatchNormOutputs HipTensorOperations::BatchNorm::calculateOutput(
        const Raw& input, const Raw& runningMean, const Raw& runningVar, const Raw& gamma, const Raw& beta) {
    const int axis = normalizeAxis(input->shape, axis_);
    const auto h = [](const Raw& t) -> uint64_t { return t ? t->storeReference : 0; };
    BatchNormOutputs r{ops_->createRaw(input->shape), ops_->createRaw({input->shape[axis]}), ops_->createRaw({input->shape[axis]})};
    check(kth_batch_norm_forward(input->storeReference, input->shape.data(), input->dimensions(), axis, training_ ? 1 : 0, momentum_,
                                 epsilon_, h(runningMean), h(runningVar), h(gamma), h(beta), r.output->storeReference,
                                 r.currentMean->storeReference, r.currentStd->storeReference));
    return r;
}
inline HipTensorOperations::BatchNormGrads HipTensorOperations::BatchNorm::calculateGrads(
        const Raw& input, const Raw& runningMean, const Raw& runningVar, const Raw& currentMean, const Raw& currentStd,
        const Raw& gamma, const Raw& gradOut, bool inRequiresGrad, bool gammaRequiresGrad, bool betaRequiresGrad) {
    BatchNormGrads r{};
    if (!inRequiresGrad && !gammaRequiresGrad && !betaRequiresGrad) return r;          // JVMBatchNorm.kt:113-115
    const int axis = normalizeAxis(input->shape, axis_);
    const auto h = [](const Raw& t) -> uint64_t { return t ? t->storeReference : 0; };
    if (inRequiresGrad) r.gradIn = ops_->createRaw(input->shape);
    if (gammaRequiresGrad) r.gradGamma = ops_->createRaw({input->shape[axis]});
    if (betaRequiresGrad) r.gradBeta = ops_->createRaw({input->shape[axis]});
    check(kth_batch_norm_backward(input->storeReference, input->shape.data(), input->dimensions(), axis, training_ ? 1 : 0, epsilon_,
                                  h(runningMean), h(runningVar), h(currentMean), h(currentStd), h(gamma), gradOut->storeReference,
                                  h(r.gradIn), h(r.gradGamma), h(r.gradBeta)));
    return r;
}
inline void HipTensorOperations::release(const Raw& t) { t->release(); }
inline void HipTensorOperations::incrementRef(const Raw& t) { t->incrementRef(); }
inline void HipTensorOperations::markSurviveGC(const Raw& t) { t->mustSurviveGC = true; }
inline void HipTensorOperations::markReleasableInGC(const Raw& t) { t->mustSurviveGC = false; }
inline void HipTensorOperations::GarbageCollector::close() {
    if (closed_ || !owner_) return;
    closed_ = true;
    ops_.collecting_ = false;
    for (const Raw& t : ops_.instances_) t->release();
    ops_.survivors_.clear();
    for (const Raw& t : ops_.instances_) if (t->referenced()) ops_.survivors_.push_back(t);
    ops_.instances_.clear();
}

// ---------------------------------------------------------------- reduce-to-shape

// functions/Utils.kt:14-41: sum(0) without keepDims once per extra leading dim, then
// sum(d, keepDims) for every remaining dim whose size differs, ascending.
inline Raw mayUnexpand(Raw rawTensor, const Shape& oldShape, HipTensorOperations& ops) {
    const int unsqueezed = rawTensor->dimensions() - static_cast<int>(oldShape.size());
    std::vector<int> expanded;
    for (size_t i = 0; i < oldShape.size(); i++)
        if (rawTensor->shape[unsqueezed + i] != oldShape[i]) expanded.push_back(static_cast<int>(i));
    Raw res = rawTensor;
    for (int i = 0; i < unsqueezed; i++) {
        Raw toRelease = res;
        res = res->sum(0, false);
        if (i > 0) ops.release(toRelease);
    }
    for (size_t i = 0; i < expanded.size(); i++) {
        Raw toRelease = res;
        res = res->sum(expanded[i], true);
        if (i > 0) ops.release(toRelease);
    }
    return res;
}

}  // namespace kten::hip
