// Drives libkten_hip.so through the C++ host mirror (include/kten_hip.hpp) on the known
// answers the reference asserts in its own suite (file:line beside each case) and on the
// error behaviour of the raw-tensor contract. Exit status 0 means every check held.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <initializer_list>

#include "kten_hip.hpp"

using namespace kten::hip;

static int g_checks = 0, g_failed = 0;

static void expect(bool ok, const char* what) {
    g_checks++;
    if (!ok) { g_failed++; std::printf("FAILED: %s\n", what); std::fflush(stdout); }
}

static void expect_values(const Raw& t, const Shape& shape, std::initializer_list<float> values, float tol, const char* what) {
    bool ok = t->shape == shape;
    const std::vector<float> got = t->toVector();
    ok = ok && got.size() == values.size();
    size_t i = 0;
    for (float v : values) { if (ok && !(std::fabs(got[i] - v) <= tol)) ok = false; i++; }
    expect(ok, what);
}

template <class F>
static void expect_illegal_argument(F&& f, const char* what) {
    bool thrown = false;
    try { f(); } catch (const std::invalid_argument&) { thrown = true; }
    expect(thrown, what);
}

static Raw tensor(HipTensorOperations& ops, const Shape& shape, std::initializer_list<float> values) {
    std::vector<float> v(values);
    return ops.createRaw(shape, [&](int i) { return v[static_cast<size_t>(i)]; });
}

int main() {
    HipTensorOperations ops(0);
    std::printf("platform: %s, %d compute units\n", ops.platformKey.c_str(), ops.computeUnits);
    std::fflush(stdout);
    {
        auto gc = ops.garbageCollector();

        // kten-testing/.../tests/TensorTestsBase.kt:33-53  [2,4] + [2,1]
        Raw t1 = tensor(ops, {2, 4}, {1, 2, 3, 4, 5, 6, 7, 8});
        Raw t2 = tensor(ops, {2, 1}, {1, 2});
        expect_values(t1->plus(t2), {2, 4}, {2, 3, 4, 5, 7, 8, 9, 10}, 0.0f, "addition with broadcast");

        // TensorTestsBase.kt:319-350  tensor - constant and constant - tensor ((-t) + c)
        Raw t3 = tensor(ops, {2, 3}, {1, 2, 3, 4, 5, 6});
        expect_values(t3->minus(2.0f), {2, 3}, {-1, 0, 1, 2, 3, 4}, 0.0f, "tensor minus constant");
        expect_values(t3->unaryMinus()->plus(2.0f), {2, 3}, {1, 0, -1, -2, -3, -4}, 0.0f, "constant minus tensor");

        // TensorTestsBase.kt:469-497  [3,3] pow [1,3]
        Raw p1 = tensor(ops, {3, 3}, {2, 3, 2, 3, 3, 3, 2, 3, 2});
        Raw p2 = tensor(ops, {1, 3}, {2, 3, 2});
        expect_values(p1->pow(p2), {3, 3}, {4, 27, 4, 9, 27, 9, 4, 27, 4}, 0.0f, "tensor pow tensor");
        // TensorTestsBase.kt:500-529  constant pow tensor
        expect_values(ops.pow(2.0f, p1), {3, 3}, {4, 8, 4, 8, 8, 8, 4, 8, 4}, 0.0f, "constant pow tensor");

        // TensorTestsBase.kt:532-609  sum / mean over an axis, with and without keepDimensions
        Raw s = tensor(ops, {3, 3}, {1, 1, 1, 2, 2, 2, 3, 3, 3});
        expect_values(s->sum(-1), {3}, {3, 6, 9}, 0.0f, "sum(axis=-1)");
        expect_values(s->sum(0, true), {1, 3}, {6, 6, 6}, 0.0f, "sum(axis=0, keepDimensions)");
        expect_values(s->mean(0), {3}, {2, 2, 2}, 0.0f, "mean(axis=0)");
        expect_values(s->mean(-1, true), {3, 1}, {1, 2, 3}, 0.0f, "mean(axis=-1, keepDimensions)");
        expect_values(s->sum(), {1}, {18}, 0.0f, "sum()");
        expect_values(s->mean(), {1}, {2}, 0.0f, "mean()");

        // TensorTestsBase.kt:612-757  max / min / argMax / argMin
        Raw m = tensor(ops, {3, 3}, {3, 2, 1, 1, 3, 2, 3, 1, 2});
        expect_values(m->max(-1), {3}, {3, 3, 3}, 0.0f, "max(axis=-1)");
        expect_values(m->min(0), {3}, {1, 1, 1}, 0.0f, "min(axis=0)");
        expect_values(m->argMax(-1), {3}, {0, 1, 0}, 0.0f, "argMax(axis=-1): ties resolve to the lowest index");
        expect_values(m->argMin(0), {3}, {1, 2, 0}, 0.0f, "argMin(axis=0)");

        // TensorTestsBase.kt:760-784  exp
        Raw e = tensor(ops, {2, 3}, {0.1f, 0.2f, 0.3f, 0.4f, 0.5f, 0.6f});
        expect_values(e->exp(), {2, 3}, {1.1052f, 1.2214f, 1.3499f, 1.4918f, 1.6487f, 1.8221f}, 1e-4f, "exp");

        // TensorTestsBase.kt:1320-1349  gather along axis 1
        Raw g = tensor(ops, {2, 2}, {1, 2, 3, 4});
        Raw gi = tensor(ops, {2, 2}, {0, 0, 1, 0});
        expect_values(g->gather(1, gi), {2, 2}, {1, 1, 4, 3}, 0.0f, "gather");

        // kten-api/.../autograd/functions/Utils.kt:14-41  reduce-to-shape of an incoming gradient
        Raw grad = ops.createRawFill({4, 3, 5}, 1.0f);
        expect_values(mayUnexpand(grad, {3, 1}, ops), {3, 1}, {20, 20, 20}, 0.0f, "mayUnexpand [4,3,5] -> [3,1]");
        expect_values(mayUnexpand(grad, {5}, ops), {5}, {12, 12, 12, 12, 12}, 0.0f, "mayUnexpand [4,3,5] -> [5]");
        Raw same = mayUnexpand(grad, {4, 3, 5}, ops);
        expect(same.get() == grad.get(), "mayUnexpand returns its argument when nothing was expanded");

        // shapes: view shares the store, reshape copies (AbstractRawTensor.kt:77-90)
        Raw v = t1->view({4, -1});
        expect(v->shape == Shape({4, 2}) && v->storeReference == t1->storeReference, "view infers -1 and shares the store");
        Raw r = t1->reshape({8});
        expect(r->shape == Shape({8}) && r->storeReference != t1->storeReference, "reshape copies");
        expect(std::fabs(t1->getSingleValue({1, -1}) - 8.0f) == 0.0f, "getSingleValue with a negative index");

        // error behaviour: IllegalArgumentException on the host side of the call
        expect_illegal_argument([&] { t1->plusAssign(t2); }, "plusAssign refuses unequal shapes (JVMRawTensor.kt:89-93)");
        expect_illegal_argument([&] { t1->plus(tensor(ops, {3}, {1, 2, 3})); }, "plus refuses shapes that do not broadcast");
        expect_illegal_argument([&] { t1->sum(2); }, "axis out of range (ShapeFunctions.kt:41-48)");
        expect_illegal_argument([&] { t1->broadcastTo({4}); }, "broadcastTo a lower rank (ShapeFunctions.kt:187-201)");
        expect_illegal_argument([&] { t1->view({3, -1, -1}); }, "view with two inferred dimensions");
        expect_illegal_argument([&] { g->gather(1, tensor(ops, {2, 2}, {0, 2, 0, 0})); }, "gather index out of range (JVMRawTensor.kt:345-346)");

        // TensorTestsBase.kt:1190-1221 transpose, :1232-1270 permute, :1272-1315 concat, :1876-1888 partial fill
        Raw tr = tensor(ops, {2, 3}, {1, 2, 3, 4, 5, 6});
        expect_values(tr->transpose(0, 1), {3, 2}, {1, 4, 2, 5, 3, 6}, 0.0f, "transpose(0, 1)");
        Raw pm = tensor(ops, {2, 3, 2}, {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12});
        expect_values(pm->permute({2, 0, 1}), {2, 2, 3}, {1, 3, 5, 7, 9, 11, 2, 4, 6, 8, 10, 12}, 0.0f, "permute(2, 0, 1)");
        Raw cat = ops.concat(0, {tensor(ops, {1, 3}, {1, 2, 3})->broadcastTo({2, 3}), tensor(ops, {1, 3}, {4, 5, 6}), tensor(ops, {1, 3}, {7, 8, 9})});
        expect_values(cat, {4, 3}, {1, 2, 3, 1, 2, 3, 4, 5, 6, 7, 8, 9}, 0.0f, "concat along axis 0");
        expect_values(cat->narrow(0, 2, 2), {2, 3}, {4, 5, 6, 7, 8, 9}, 0.0f, "narrow");
        Raw pf = ops.createRawFill({2, 3}, 2.0f);
        pf->set(std::vector<IntRange>{{0, 0}, {1, 2}}, 0.0f);
        expect_values(pf, {2, 3}, {2, 0, 0, 2, 2, 2}, 0.0f, "set(ranges, Float)");
        // TensorTestsBase.kt:152-188: t2[1..1, all, 1..-1] = value of shape [1, 3, 2]
        Raw big = ops.createRawFill({3, 3, 3}, 1.0f);
        big->set(std::vector<IntRange>{{1, 1}, All, {1, -1}}, ops.createRawFill({1, 3, 2}, 0.01f));
        expect_values(big->get(std::vector<int>{1}), {3, 3}, {1, 0.01f, 0.01f, 1, 0.01f, 0.01f, 1, 0.01f, 0.01f}, 0.0f, "set(ranges, tensor) and get(IntArray)");
        expect_values(big->get(std::vector<IntRange>{All, {0, 0}, {2, 2}}), {3, 1, 1}, {1, 0.01f, 1}, 0.0f, "get(ranges)");
        expect_values(tr->maskedFill(tensor(ops, {3}, {1, 0, 1}), -1.0f), {2, 3}, {-1, 2, -1, -1, 5, -1}, 0.0f, "maskedFill with a broadcast mask");
        expect_illegal_argument([&] { big->get(std::vector<IntRange>{{2, 1}}); }, "range with first > last");
        expect_illegal_argument([&] { big->set(std::vector<IntRange>{{0, 0}}, ops.createRawFill({2}, 1.0f)); }, "set(ranges) with a different element count");
        expect_illegal_argument([&] { pm->permute({0, 0, 1}); }, "permute must name every axis");
        expect_illegal_argument([&] { tr->transpose(1, -1); }, "transpose needs two different axes");

        // BatchNormOperation, inference mode (TensorTestsBase.kt:2064-2084): (x - mean) / sqrt(var + eps) * gamma + beta
        Raw bx = tensor(ops, {2, 2, 2}, {1, 2, 3, 4, 5, 6, 7, 8});
        Raw bmean = tensor(ops, {2}, {1, 3}), bvar = tensor(ops, {2}, {3, 15}), bgamma = tensor(ops, {2}, {2, 4}), bbeta = tensor(ops, {2}, {1, -1});
        auto bn = ops.batchNorm(1, 0.1f, 1.0f, false).calculateOutput(bx, bmean, bvar, bgamma, bbeta);
        expect_values(bn.output, {2, 2, 2}, {1, 2, -1, 0, 5, 6, 3, 4}, 0.0f, "batchNorm inference: exact for var + eps = 4 and 16");
        // training mode: channel mean and the reciprocal standard deviation (biased variance 4.25, eps 0)
        auto bt = ops.batchNorm(1, 0.1f, 0.0f, true).calculateOutput(bx, nullptr, nullptr, nullptr, nullptr);
        expect_values(bt.currentMean, {2}, {3.5f, 5.5f}, 0.0f, "batchNorm training: channel means");
        expect_values(bt.currentStd, {2}, {0.48507125f, 0.48507125f}, 1e-7f, "batchNorm training: 1 / sqrt(var)");
        auto bg = ops.batchNorm(1, 0.1f, 0.0f, true).calculateGrads(bx, nullptr, nullptr, bt.currentMean, bt.currentStd, nullptr,
                                                                    ops.createRawFill({2, 2, 2}, 1.0f), true, false, true);
        expect_values(bg.gradBeta, {2}, {4, 4}, 0.0f, "batchNorm gradBeta = sum of gradOut");
        expect_values(bg.gradIn, {2, 2, 2}, {0, 0, 0, 0, 0, 0, 0, 0}, 1e-6f, "batchNorm gradIn of a constant gradient is zero");
        expect(bg.gradGamma == nullptr, "a gradient that is not required is not produced");
        expect_illegal_argument([&] { ops.batchNorm(1, 0.1f, 1e-3f, false).calculateOutput(bx, nullptr, nullptr, nullptr, nullptr); },
                                "inference mode needs running statistics");

        // in-place arithmetic and NaN detection
        Raw acc = ops.zerosLike(t1);
        acc->plusAssign(t1);
        acc->timesAssign(2.0f);
        acc->plusAssign(1.0f);
        expect_values(acc, {2, 4}, {3, 5, 7, 9, 11, 13, 15, 17}, 0.0f, "plusAssign / timesAssign");
        expect(!acc->containsNan(), "containsNan on finite values");
        expect(tensor(ops, {2}, {1.0f, NAN})->containsNan(), "containsNan finds a NaN");

        // inplaceResize keeps the leading values and pads with zeros; a shallow copy keeps the old store
        Raw grown = tensor(ops, {3}, {1, 2, 3});
        Raw alias = grown->copy(true);
        grown->inplaceResize({2, 3});
        expect_values(grown, {2, 3}, {1, 2, 3, 0, 0, 0}, 0.0f, "inplaceResize grows with zeros");
        grown->inplaceResize({2});
        expect_values(grown, {2}, {1, 2}, 0.0f, "inplaceResize truncates");
        expect_values(alias, {3}, {1, 2, 3}, 0.0f, "a shallow copy still sees the store it shares");

        // survive the scope
        ops.markSurviveGC(t1);
        gc.close();
        expect(t1->referenced() && !t2->referenced(), "garbage collector scope releases all but the survivors");
        ops.markReleasableInGC(t1);
        t1->release();
    }
    {
        // The math mode: exact gives the float of the f64 routine (what kotlin.math's Float overloads return), the
        // default stays within one ulp of it on these values; a copy is the source's values whoever is written next
        // (the library puts the copy off until then).
        auto gc = ops.garbageCollector();
        std::vector<float> xs;
        for (int i = 0; i < 4096; i++) xs.push_back(-6.0f + 12.0f * static_cast<float>(i) / 4095.0f);
        Raw x = ops.createRaw({4096}, [&](int i) { return xs[static_cast<size_t>(i)]; });
        expect(ops.getMathMode() == HipTensorOperations::MathMode::WITHIN_2_ULP, "the default math mode is within two ulp");
        const std::vector<float> fast = x->tanh()->toVector();
        ops.setMathMode(HipTensorOperations::MathMode::EXACT);
        const std::vector<float> exact = x->tanh()->toVector();
        ops.setMathMode(HipTensorOperations::MathMode::WITHIN_2_ULP);
        bool exact_ok = true, fast_ok = true;
        for (size_t i = 0; i < xs.size(); i++) {
            const float want = static_cast<float>(std::tanh(static_cast<double>(xs[i])));
            if (exact[i] != want) exact_ok = false;
            if (!(std::fabs(fast[i] - want) <= std::fabs(std::nextafter(want, 2.0f) - want))) fast_ok = false;
        }
        expect(exact_ok, "tanh in mode exact is the rounded f64 tanh");
        expect(fast_ok, "tanh in the default mode is within one ulp of it");
        Raw c = x->copy();
        Raw p = x->pow(1.0f);
        x->timesAssign(2.0f);
        const std::vector<float> cv = c->toVector(), pv = p->toVector(), xv = x->toVector();
        bool kept = true;
        for (size_t i = 0; i < xs.size(); i++) if (cv[i] != xs[i] || pv[i] != xs[i] || xv[i] != 2.0f * xs[i]) kept = false;
        expect(kept, "copy() and pow(1) keep the source's values when the source is written afterwards");
    }
    {
        // The chain of the autograd reduce-to-shape ([64,40,100] -> [64,100] -> [64], each intermediate released after the
        // next sum, Utils.kt:26-38): whole numbers, so that every order of adding gives the same float. The library puts
        // the first sum off and runs both in the second call's launch; the source may be written or released in between.
        auto gc = ops.garbageCollector();
        Raw x = ops.createRaw({64, 40, 100}, [](int i) { return static_cast<float>(i % 7 - 3); });
        const std::vector<float> xs = x->toVector();
        std::vector<float> rows(64 * 100, 0.0f), totals(64, 0.0f);
        for (int o = 0; o < 64; o++)
            for (int a = 0; a < 40; a++)
                for (int i = 0; i < 100; i++) {
                    rows[static_cast<size_t>(o * 100 + i)] += xs[static_cast<size_t>((o * 40 + a) * 100 + i)];
                    totals[static_cast<size_t>(o)] += xs[static_cast<size_t>((o * 40 + a) * 100 + i)];
                }
        Raw first = x->sum(1, false);
        Raw second = first->sum(1, false);
        first->release();
        expect(second->toVector() == totals, "two steps of a reduce-to-shape chain");
        Raw kept = x->sum(1, false);
        x->timesAssign(0.0f);                           // the sum is that of the values at the call
        x->release();
        expect(kept->toVector() == rows, "a sum whose source is written and released before anybody reads it");
    }
    std::printf("%d checks, %d failed\n", g_checks, g_failed);
    return g_failed == 0 ? 0 : 1;
}
