/*
 * TEST INFRASTRUCTURE ONLY -- thin extern "C" window onto the parts of the reference that build
 * without its third-party dependencies: the Clifford sign tables and product iterators
 * (src/algebras.{hpp,cc}) and the environment-switch parsing of Context (src/backend/backend.{hpp,cc}).
 * Compiled by oracle/build.py against the reference sources where they lie; the result goes to
 * oracle/_ref/ and is used only to validate the restatement in qoracle.c.
 * The rest of the reference's CPU path needs oneDNN (absent) and is not buildable here.
 */
#include "algebras.hpp"
#include "backend/backend.hpp"

using namespace upstride;

namespace {
struct OpenContext : public Context {
    OpenContext() : Context() {}
};

template <int A>
int dumpTable(int* left, int* right, int* positive, int* layout, int* order) {
    using Spec = CliffordProductSpec<A>;
    const int total = Spec::SIGNTABLE_LAYOUT[Spec::DIMS];
    for (int i = 0; i < total; ++i) {
        left[i] = Spec::SIGNTABLE[i].left;
        right[i] = Spec::SIGNTABLE[i].right;
        positive[i] = Spec::SIGNTABLE[i].positive ? 1 : 0;
        order[i] = Spec::BACKPROP_ORDER[i];
    }
    for (int i = 0; i <= Spec::DIMS; ++i) layout[i] = Spec::SIGNTABLE_LAYOUT[i];
    return Spec::DIMS;
}

template <int A>
int dumpTerms(bool backprop, int* out) {
    int k = 0;
    auto fill = [&](int l, int r, int d) {
        out[5 * k + 0] = l; out[5 * k + 1] = r; out[5 * k + 2] = d; out[5 * k + 3] = 1; out[5 * k + 4] = 1;
        ++k;
    };
    auto acc = [&](int l, int r, int d, bool positive) {
        out[5 * k + 0] = l; out[5 * k + 1] = r; out[5 * k + 2] = d; out[5 * k + 3] = positive ? 1 : 0; out[5 * k + 4] = 0;
        ++k;
    };
    if (backprop)
        BinaryOperation<CliffordProductSpec<A>>::productBackprop(fill, acc);
    else
        BinaryOperation<CliffordProductSpec<A>>::product(fill, acc);
    return k;
}
}  // namespace

extern "C" {

int ref_multivector_dim(int algebra) { return MULTIVECTOR_DIM[algebra]; }

int ref_sign_table(int algebra, int* left, int* right, int* positive, int* layout, int* order) {
    switch (algebra) {
        case REAL: return dumpTable<REAL>(left, right, positive, layout, order);
        case COMPLEX: return dumpTable<COMPLEX>(left, right, positive, layout, order);
        case QUATERNION: return dumpTable<QUATERNION>(left, right, positive, layout, order);
        case GA_300: return dumpTable<GA_300>(left, right, positive, layout, order);
    }
    return -1;
}

/* out receives 5 ints per term: left, right, dim, positive, fill */
int ref_terms(int algebra, int backprop, int* out) {
    try {
        switch (algebra) {
            case REAL: return dumpTerms<REAL>(backprop != 0, out);
            case COMPLEX: return dumpTerms<COMPLEX>(backprop != 0, out);
            case QUATERNION: return dumpTerms<QUATERNION>(backprop != 0, out);
            case GA_300: return dumpTerms<GA_300>(backprop != 0, out);
        }
    } catch (...) {
    }
    return -1;
}

/* reads UPSTRIDE_MEMORY_OPTIMIZED / UPSTRIDE_CONV_FP16_POLICY from the process environment */
void ref_context_switches(int* preferSpeedToMemory, int* fp16Forward, int* fp16Backward) {
    OpenContext ctx;
    *preferSpeedToMemory = ctx.preferSpeedToMemory() ? 1 : 0;
    *fp16Forward = ctx.isFp16ConvForwardAllowed() ? 1 : 0;
    *fp16Backward = ctx.isFp16ConvBackwardAllowed() ? 1 : 0;
}

int ref_algebra_from_type(int uptype) {
    try {
        return getAlgebraFromType(uptype);
    } catch (const std::invalid_argument&) {
        return -1;
    }
}
}
