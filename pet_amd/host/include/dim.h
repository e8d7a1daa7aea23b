// Shapes and index ranges (role of the reference's include/dim.h).
#pragma once
#include <algorithm>
#include <cassert>
#include <string>
#include <vector>

namespace tpm {

using Dim = std::vector<int>;

template <class F> inline Dim zipDims(const Dim &a, const Dim &b, F f) {
    assert(a.size() == b.size());
    Dim out(a.size());
    for (size_t i = 0; i < a.size(); ++i)
        out[i] = f(a[i], b[i]);
    return out;
}
inline Dim elementwiseMin(const Dim &a, const Dim &b) {
    return zipDims(a, b, [](int x, int y) { return std::min(x, y); });
}
inline Dim elementwiseMax(const Dim &a, const Dim &b) {
    return zipDims(a, b, [](int x, int y) { return std::max(x, y); });
}
inline Dim elementwiseAdd(const Dim &a, const Dim &b) {
    return zipDims(a, b, [](int x, int y) { return x + y; });
}
inline Dim elementwiseSub(const Dim &a, const Dim &b) {
    return zipDims(a, b, [](int x, int y) { return x - y; });
}

inline std::string dimToString(const Dim &d) {
    std::string s = "[";
    for (size_t i = 0; i < d.size(); ++i)
        s += (i ? "," : "") + std::to_string(d[i]);
    return s + "]";
}

inline size_t dimProduct(const Dim &d) {
    size_t p = 1;
    for (int v : d)
        p *= (size_t)v;
    return p;
}

// Row-major linear index -> index vector (include/dim.h:60-70).
inline Dim cntToIdx(const Dim &dim, size_t cnt) {
    Dim idx(dim.size(), 0);
    for (int j = (int)dim.size() - 1; j >= 0 && cnt > 0; --j) {
        idx[j] = (int)(cnt % (size_t)dim[j]);
        cnt /= (size_t)dim[j];
    }
    return idx;
}

// A closed box of positions, or one of the symbolic ranges All / Empty
// (include/dim.h:72-135).
class DimRange {
    enum State { AllPos, Empty, SinglePos, RangePos, Invalid };
    Dim begin, end;
    State state;
    explicit DimRange(State s) : state(s) {}

  public:
    DimRange() : state(Invalid) {}
    DimRange(const Dim &point) : begin(point), end(point), state(point.empty() ? Invalid : SinglePos) {}
    DimRange(const Dim &b, const Dim &e) : begin(b), end(e), state(Invalid) {
        if (b.empty() || b.size() != e.size())
            return;
        bool single = true;
        for (size_t i = 0; i < b.size(); ++i) {
            if (b[i] > e[i])
                return;
            single = single && b[i] == e[i];
        }
        state = single ? SinglePos : RangePos;
    }
    Dim &getBegin() { return begin; }
    const Dim &getBegin() const { return begin; }
    Dim &getEnd() { return end; }
    const Dim &getEnd() const { return end; }
    bool isSinglePos() const { return state == SinglePos; }
    bool isEmpty() const { return state == Empty; }
    bool isAllPos() const { return state == AllPos; }
    bool notValid() const { return state == Invalid; }
    bool valid() const { return state != Invalid; }
    static DimRange getInvalid() { return DimRange(Invalid); }
    static DimRange getEmpty() { return DimRange(Empty); }
    static DimRange getAllPos() { return DimRange(AllPos); }
};

inline DimRange unionRange(const DimRange &a, const DimRange &b) {
    if (a.notValid() || b.notValid())
        return DimRange::getInvalid();
    if (a.isAllPos() || b.isAllPos())
        return DimRange::getAllPos();
    if (a.isEmpty())
        return b;
    if (b.isEmpty())
        return a;
    return DimRange(elementwiseMin(a.getBegin(), b.getBegin()),
                    elementwiseMax(a.getEnd(), b.getEnd()));
}

} // namespace tpm
