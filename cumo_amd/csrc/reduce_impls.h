// Reduction semantics: what each reduction folds and how accumulators merge.
//
// The rules are the reference's impl structs
// (ext/cumo/narray/gen/tmpl/real_accum_kernel.cu:11-157,
// float_accum_kernel.cu:15-146, accum_arg_kernel.cu:15-112,
// accum_index_kernel.cu:15-112), which in turn restate Numo's sequential loops
// (ext/cumo/include/cumo/types/real_accum.h:25-441): NaN skipping, all-NaN
// answers, lowest index on ties, Int32 sums widening to 64 bits.
//
// Every combine() is insensitive to the order in which accumulators arrive,
// so the kernels are free to interleave lanes. Where Numo's answer depends on
// order -- which of two equal elements min/max keep, i.e. the sign of a zero --
// the accumulator carries the index and the earlier element wins, as the
// reference's tests require (test/narray_test.rb:667-672).
#ifndef CUMO_HIP_REDUCE_IMPLS_H
#define CUMO_HIP_REDUCE_IMPLS_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>
#include <float.h>

namespace cumo_hip {

template <class T> struct is_float_t { static constexpr bool value = false; };
template <> struct is_float_t<float> { static constexpr bool value = true; };
template <> struct is_float_t<double> { static constexpr bool value = true; };

template <class T> __device__ __forceinline__ bool isnan_t(T x) { return x != x; }
template <> __device__ __forceinline__ bool isnan_t<int32_t>(int32_t) { return false; }

// what an accumulator of min/max starts from: `skip` loses to every element
// (NaN for floats), `lowest`/`highest` lose to every element but a NaN
template <class T> struct Lim;
template <> struct Lim<float> {
    static __device__ __forceinline__ float skip() { return __int_as_float(0x7fc00000); }
    static __device__ __forceinline__ float highest() { return __int_as_float(0x7f800000); }
    static __device__ __forceinline__ float lowest() { return __int_as_float(0xff800000); }
};
template <> struct Lim<double> {
    static __device__ __forceinline__ double skip() { return __longlong_as_double(0x7ff8000000000000ll); }
    static __device__ __forceinline__ double highest() { return __longlong_as_double(0x7ff0000000000000ll); }
    static __device__ __forceinline__ double lowest() { return __longlong_as_double(0xfff0000000000000ll); }
};
template <> struct Lim<int32_t> {
    static __device__ __forceinline__ int32_t skip() { return 0; }
    static __device__ __forceinline__ int32_t highest() { return INT32_MAX; }
    static __device__ __forceinline__ int32_t lowest() { return INT32_MIN; }
};

template <class T> __device__ __forceinline__ T spread(T hi, T lo) { return hi - lo; }
template <> __device__ __forceinline__ int32_t spread<int32_t>(int32_t hi, int32_t lo) { return (int32_t)((uint32_t)hi - (uint32_t)lo); }

// the plain element-by-element form of accumulate_n
#define CUMO_HIP_ACCUMULATE_N_BY_ELEMENT                                                          \
    template <int N>                                                                              \
    __device__ __forceinline__ void accumulate_n(const In (&x)[N], int64_t idx0, Acc& acc) const { \
        _Pragma("unroll") for (int k = 0; k < N; ++k) accumulate(x[k], idx0 + k, acc);            \
    }

// The hardware's max/min: of a number and a quiet NaN the number is kept. One
// instruction each; the C library's fmax/fmin cost three here, because the
// compiler quiets both operands first. A signalling NaN comes out as a NaN, which
// the callers treat as "look at this block element by element".
template <class T> __device__ __forceinline__ T max_skipping_nan(T a, T b);
template <> __device__ __forceinline__ float max_skipping_nan<float>(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
template <> __device__ __forceinline__ double max_skipping_nan<double>(double a, double b) {
    double r;
    asm("v_max_f64 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
template <> __device__ __forceinline__ int32_t max_skipping_nan<int32_t>(int32_t a, int32_t b) { return a > b ? a : b; }
template <class T> __device__ __forceinline__ T min_skipping_nan(T a, T b);
template <> __device__ __forceinline__ float min_skipping_nan<float>(float a, float b) {
    float r;
    asm("v_min_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
template <> __device__ __forceinline__ double min_skipping_nan<double>(double a, double b) {
    double r;
    asm("v_min_f64 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
template <> __device__ __forceinline__ int32_t min_skipping_nan<int32_t>(int32_t a, int32_t b) { return a < b ? a : b; }

// true if any of the N values is a NaN (a sum is NaN then; inf - inf also trips
// it, which only costs the slow path)
template <class T, int N>
__device__ __forceinline__ bool maybe_nan(const T (&x)[N]) {
    if (!is_float_t<T>::value) return false;
    T s = x[0];
#pragma unroll
    for (int k = 1; k < N; ++k) s = s + x[k];
    return s != s;
}

// ---- sum / prod / mean -------------------------------------------------------
// TA: accumulator type (the input type for floats, int64 for Int32:
// narray/gen/spec.rb:308-319). divisor != 0 turns the sum into a mean
// (float_accum_kernel.cu:42-50).
template <class T, class TA, bool PROD, bool SKIP_NAN>
struct SumImpl {
    typedef T In;
    typedef TA Acc;
    static constexpr bool USES_INDEX = false;
    static constexpr int NOUT = 1;
    TA divisor;
    // results have the input's type: a reduction may go through results of its own (rows first, then the rows' results),
    // the division only at the end
    static constexpr bool OWN_RESULTS = sizeof(T) == sizeof(TA);
    SumImpl before_the_last() const { return SumImpl{(TA)0}; }
    __device__ __forceinline__ Acc identity() const { return PROD ? (TA)1 : (TA)0; }
    __device__ __forceinline__ void accumulate(T x, int64_t, Acc& acc) const {
        if (SKIP_NAN && isnan_t(x)) return;
        if (PROD) acc = (TA)x * acc; else acc = (TA)x + acc;
    }
    CUMO_HIP_ACCUMULATE_N_BY_ELEMENT
    __device__ __forceinline__ void combine(const Acc& next, Acc& acc) const {
        if (PROD) acc = next * acc; else acc = next + acc;
    }
    __device__ __forceinline__ void store(const Acc& acc, char* out, char*) const {
        *reinterpret_cast<TA*>(out) = (divisor != (TA)0) ? (TA)(acc / divisor) : acc;
    }
};

// mean(nan: true): the count of what was left rides along (float_accum_kernel.cu:86-101)
template <class T>
struct MeanNanImpl {
    typedef T In;
    struct Acc { T sum; int64_t n; };
    static constexpr bool USES_INDEX = false;
    static constexpr int NOUT = 1;
    __device__ __forceinline__ Acc identity() const { return Acc{(T)0, 0}; }
    __device__ __forceinline__ void accumulate(T x, int64_t, Acc& acc) const {
        if (isnan_t(x)) return;
        acc.sum = x + acc.sum;
        acc.n += 1;
    }
    CUMO_HIP_ACCUMULATE_N_BY_ELEMENT
    __device__ __forceinline__ void combine(const Acc& next, Acc& acc) const { acc.sum = next.sum + acc.sum; acc.n += next.n; }
    __device__ __forceinline__ void store(const Acc& acc, char* out, char*) const { *reinterpret_cast<T*>(out) = acc.sum / (T)acc.n; }
};

// ---- rms ----------------------------------------------------------------------
// count: the length of the reduce axis, known to the launcher
// (float_accum_kernel.cu:52-58); the nan form counts what it kept (:103-116).
template <class T, bool SKIP_NAN>
struct RmsImpl {
    typedef T In;
    // (the count rides along only where NaNs are skipped: otherwise it is the axis' length, and the accumulator is
    // as small as the sum's)
    struct Counted { T sum; int64_t n; };
    struct Plain { T sum; };
    typedef typename std::conditional<SKIP_NAN, Counted, Plain>::type Acc;
    static constexpr bool USES_INDEX = false;
    static constexpr int NOUT = 1;
    T count;
    __device__ __forceinline__ Acc identity() const { Acc a = Acc(); a.sum = (T)0; return a; }
    __device__ __forceinline__ void accumulate(T x, int64_t, Acc& acc) const {
        if constexpr (SKIP_NAN) {
            if (isnan_t(x)) return;
            acc.n += 1;
        }
        acc.sum += x * x;
    }
    CUMO_HIP_ACCUMULATE_N_BY_ELEMENT
    __device__ __forceinline__ void combine(const Acc& next, Acc& acc) const {
        acc.sum += next.sum;
        if constexpr (SKIP_NAN) acc.n += next.n;
    }
    __device__ __forceinline__ void store(const Acc& acc, char* out, char*) const {
        T n = count;
        if constexpr (SKIP_NAN) n = (T)acc.n;
        *reinterpret_cast<T*>(out) = (T)sqrt((double)(acc.sum / n));
    }
};

// ---- var / stddev: Welford per element, Chan between accumulators ---------------
// (float_accum_kernel.cu:10-40,102-125). Numo takes two passes with the exact
// mean (types/real_accum.h:114-131); the two agree to rounding.
template <class T, bool SKIP_NAN>
struct MomentsImpl {
    typedef T In;
    struct Acc { T n; T mean; T m2; };
    static constexpr bool USES_INDEX = false;
    static constexpr int NOUT = 1;
    int take_sqrt;
    __device__ __forceinline__ Acc identity() const { return Acc{(T)0, (T)0, (T)0}; }
    __device__ __forceinline__ void accumulate(T x, int64_t, Acc& acc) const {
        if (SKIP_NAN && isnan_t(x)) return;
        acc.n += (T)1;
        const T delta = x - acc.mean;
        acc.mean += delta / acc.n;
        acc.m2 += delta * (x - acc.mean);
    }
    __device__ __forceinline__ void combine(const Acc& next, Acc& acc) const {
        if (next.n == (T)0) return;
        if (acc.n == (T)0) { acc = next; return; }
        const T n = acc.n + next.n;
        const T delta = next.mean - acc.mean;
        // equal counts (every step of the combine across lanes that hold equal shares): no division
        const T w = (next.n == acc.n) ? (T)0.5 : next.n / n;
        acc.mean = acc.mean + delta * w;
        acc.m2 += next.m2 + delta * delta * acc.n * w;
        acc.n = n;
    }
    // N elements at once: their own mean and squared deviations in two passes over
    // registers (no division: N is a power of two), then one Chan merge. One
    // division per N elements instead of one per element, and the block statistics
    // are as accurate as Numo's own two-pass form.
    template <int N>
    __device__ __forceinline__ void accumulate_n(const T (&x)[N], int64_t idx0, Acc& acc) const {
        if (N == 1 || (N & (N - 1)) != 0 || (SKIP_NAN && maybe_nan<T, N>(x))) {
#pragma unroll
            for (int k = 0; k < N; ++k) accumulate(x[k], idx0 + k, acc);
            return;
        }
        T s = x[0];
#pragma unroll
        for (int k = 1; k < N; ++k) s = s + x[k];
        const T mb = s * ((T)1 / (T)N);
        T m2 = (T)0;
#pragma unroll
        for (int k = 0; k < N; ++k) {
            const T d = x[k] - mb;
            m2 = m2 + d * d;
        }
        combine(Acc{(T)N, mb, m2}, acc);
    }
    // U positions of VEC neighbouring outputs at once (the column form: a lane's outputs have all seen the same
    // number of positions): each output's own two passes over its U values, and one merge each with the ONE weight
    // U / (n + U) that the count gives all of them (one division a step instead of one an output).
    static constexpr bool COLUMNS_TOGETHER = !SKIP_NAN;
    template <int U, int VEC>
    __device__ __forceinline__ void accumulate_columns(const T (&x)[U][VEC], Acc (&acc)[VEC]) const {
        const T n = acc[0].n;
        const T n_new = n + (T)U;
        const T w = (T)U / n_new;
        const T nw = n * w;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            T s = x[0][j];
#pragma unroll
            for (int u = 1; u < U; ++u) s = s + x[u][j];
            const T mb = s * ((T)1 / (T)U);
            T m2 = (T)0;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const T d = x[u][j] - mb;
                m2 = m2 + d * d;
            }
            const T delta = mb - acc[j].mean;
            acc[j].mean = acc[j].mean + delta * w;
            acc[j].m2 += m2 + delta * delta * nw;
            acc[j].n = n_new;
        }
    }
    // U blocks of N at once: the same two passes over all U * N values, one merge (and one
    // division) for all of them.
    static constexpr bool GROUPED = true;
    template <int U, int N>
    __device__ __forceinline__ void accumulate_group(const T (&x)[U][N], const int64_t (&idx)[U], Acc& acc) const {
        constexpr int M = U * N;
        bool plain = (M & (M - 1)) != 0;
        if (SKIP_NAN && !plain) {
#pragma unroll
            for (int u = 0; u < U; ++u) plain = plain || maybe_nan<T, N>(x[u]);
        }
        if (plain) {
#pragma unroll
            for (int u = 0; u < U; ++u) accumulate_n<N>(x[u], idx[u], acc);
            return;
        }
        T part[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            part[u] = x[u][0];
#pragma unroll
            for (int k = 1; k < N; ++k) part[u] = part[u] + x[u][k];
        }
        T s = part[0];
#pragma unroll
        for (int u = 1; u < U; ++u) s = s + part[u];
        const T mb = s * ((T)1 / (T)M);
        T q[U];   // one chain of additions per vector, so that they run side by side
#pragma unroll
        for (int u = 0; u < U; ++u) {
            q[u] = (T)0;
#pragma unroll
            for (int k = 0; k < N; ++k) {
                const T d = x[u][k] - mb;
                q[u] = q[u] + d * d;
            }
        }
        T m2 = q[0];
#pragma unroll
        for (int u = 1; u < U; ++u) m2 = m2 + q[u];
        combine(Acc{(T)M, mb, m2}, acc);
    }
    __device__ __forceinline__ void store(const Acc& acc, char* out, char*) const {
        // every element NaN leaves no count; Numo answers +0 there (float_accum_kernel.cu:74-84)
        T v = (SKIP_NAN && acc.n == (T)0) ? (T)0 : acc.m2 / (acc.n - (T)1);
        if (take_sqrt) v = (T)sqrt((double)v);
        *reinterpret_cast<T*>(out) = v;
    }
};

// ---- kahan_sum (DFloat): Neumaier partials (float_accum_kernel.cu:116-146) ------
template <class T, bool SKIP_NAN>
struct KahanImpl {
    typedef T In;
    struct Acc { T sum; T comp; };
    static constexpr bool USES_INDEX = false;
    static constexpr int NOUT = 1;
    __device__ __forceinline__ Acc identity() const { return Acc{(T)0, (T)0}; }
    __device__ __forceinline__ void combine(const Acc& next, Acc& acc) const {
        const T t = acc.sum + next.sum;
        const T c = (fabs(acc.sum) >= fabs(next.sum)) ? (acc.sum - t) + next.sum : (next.sum - t) + acc.sum;
        acc.comp += next.comp + c;
        acc.sum = t;
    }
    __device__ __forceinline__ void accumulate(T x, int64_t, Acc& acc) const {
        if (SKIP_NAN && isnan_t(x)) return;
        combine(Acc{x, (T)0}, acc);
    }
    CUMO_HIP_ACCUMULATE_N_BY_ELEMENT
    __device__ __forceinline__ void store(const Acc& acc, char* out, char*) const { *reinterpret_cast<T*>(out) = acc.sum + acc.comp; }
};

// ---- min / max / argmin / argmax / min_index / max_index -------------------------
// One accumulator for all of them: the value and the index it was seen at.
// NAN_WINS = false: a NaN loses to anything, every element NaN answers the first
// (accum_arg_kernel.cu:15-37). NAN_WINS = true (nan: true): the first NaN wins
// outright (accum_arg_kernel.cu:40-61). Equal values: lower index.
// out_mode: 0 store the value (min/max), 4 / 8 store the index as int32 / int64.
// IDX: the type the index is kept in while folding (int32_t halves a 4-byte type's accumulator and
// the traffic between lanes; the launcher picks it when every index fits).
template <class T, bool IS_MAX, bool NAN_WINS, class IDX = int64_t>
struct ArgImpl {
    typedef T In;
    struct Acc { T value; IDX index; };
    static constexpr IDX kNone = sizeof(IDX) == 8 ? (IDX)INT64_MAX : (IDX)INT32_MAX;  // no element seen yet
    static constexpr bool USES_INDEX = true;
    static constexpr int NOUT = 1;
    int out_mode;
    __device__ __forceinline__ Acc identity() const {
        if (is_float_t<T>::value && !NAN_WINS) return Acc{Lim<T>::skip(), kNone};
        return Acc{IS_MAX ? Lim<T>::lowest() : Lim<T>::highest(), kNone};
    }
    __device__ __forceinline__ void combine(const Acc& next, Acc& acc) const {
        if (is_float_t<T>::value) {
            const bool an = isnan_t(acc.value), nn = isnan_t(next.value);
            if (an || nn) {
                if (NAN_WINS) {
                    if (nn && (!an || next.index < acc.index)) acc = next;
                } else {
                    if (an && (!nn || next.index < acc.index)) acc = next;
                }
                return;
            }
        }
        const bool better = IS_MAX ? (acc.value < next.value) : (acc.value > next.value);
        if (better || (acc.value == next.value && next.index < acc.index)) acc = next;
    }
    __device__ __forceinline__ void accumulate(T x, int64_t idx, Acc& acc) const { combine(Acc{x, (IDX)idx}, acc); }
    // (an accumulator of the value-only form this is the exact rule of: a plain value, folded as an element at position idx)
    __device__ __forceinline__ void accumulate_acc(T part, int64_t idx, Acc& acc) const { accumulate(part, idx, acc); }
    // N later elements at once. The block's extreme costs one max/min per element;
    // only a block that beats the accumulator is looked at again, to find where its
    // extreme first occurs, and then merged with one combine. An equal value never
    // replaces, because everything in the block is later than what the accumulator
    // holds.
    template <int N>
    __device__ __forceinline__ void accumulate_n(const T (&x)[N], int64_t idx0, Acc& acc) const {
        if (N == 1) {
            accumulate(x[0], idx0, acc);
            return;
        }
        T m = x[0];
#pragma unroll
        for (int k = 1; k < N; ++k) m = IS_MAX ? max_skipping_nan<T>(m, x[k]) : min_skipping_nan<T>(m, x[k]);
        if (is_float_t<T>::value && !NAN_WINS) {
            // One ordered comparison settles the common case. It is false, and the
            // block gets looked at, when the block's extreme is better, when the
            // accumulator holds nothing but NaN so far, and when m came out a NaN.
            if (IS_MAX ? (m <= acc.value) : (m >= acc.value)) return;
            if (isnan_t(m)) {  // all NaN, or a signalling NaN poisoned m: exact rule, element by element
#pragma unroll
                for (int k = 0; k < N; ++k) accumulate(x[k], idx0 + k, acc);
                return;
            }
        } else {
            bool look = IS_MAX ? (m > acc.value) : (m < acc.value);
            look = look || acc.index == kNone;
            if (is_float_t<T>::value) {  // NAN_WINS
                if (isnan_t(acc.value)) return;  // an earlier NaN already won
                if (maybe_nan<T, N>(x)) {         // rare: let the exact rule sort it out
#pragma unroll
                    for (int k = 0; k < N; ++k) accumulate(x[k], idx0 + k, acc);
                    return;
                }
            }
            if (!look) return;
        }
        // first position holding the extreme; if every element is a NaN, m is one and
        // nothing compares equal, which leaves the block's first element
        // (the value is taken from that position too: of +0 and -0 the earlier counts)
        int first = 0;
        T v = is_float_t<T>::value ? x[0] : m;
#pragma unroll
        for (int k = N - 1; k >= 0; --k) {
            const bool hit = x[k] == m;
            first = hit ? k : first;
            v = hit ? x[k] : v;
        }
        combine(Acc{v, (IDX)(idx0 + first)}, acc);
    }
    // U consecutive positions (idx0, idx0 + 1, ...) of N neighbouring outputs, every position later than what the
    // accumulators hold, without a branch: the column kernels' lanes each have outputs of their own, and with a test
    // per output some lane of the wave nearly always takes the long way. What combine() decides for a later
    // element: a better number wins; a NaN wins over a number (NAN_WINS) or loses to it; nothing seen yet loses to anything.
    static constexpr bool COLUMNS_BY_POSITION = true;
    template <int U, int N>
    __device__ __forceinline__ void accumulate_columns_by_position(const T (&x)[U][N], int64_t idx0, Acc (&acc)[N]) const {
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int j = 0; j < N; ++j) {
                const T v = x[u][j];
                const bool better = IS_MAX ? (acc[j].value < v) : (acc[j].value > v);   // false with a NaN on either side
                const bool first = acc[j].index == kNone;
                bool take;
                if (is_float_t<T>::value) {
                    const bool an = isnan_t(acc[j].value), nn = isnan_t(v);
                    take = NAN_WINS ? (better || (nn && !an) || first) : (better || (an && (!nn || first)));
                } else {
                    take = better || first;
                }
                acc[j].value = take ? v : acc[j].value;
                acc[j].index = take ? (IDX)(idx0 + u) : acc[j].index;
            }
        }
    }
    // U blocks of N at once (all later than what the accumulator holds): when no
    // element of any of them can change the accumulator, one comparison says so.
    static constexpr bool GROUPED = true;
    template <int U, int N>
    __device__ __forceinline__ void accumulate_group(const T (&x)[U][N], const int64_t (&idx)[U], Acc& acc) const {
        if (!is_float_t<T>::value || !NAN_WINS) {
            T m = x[0][0];
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
                for (int k = 0; k < N; ++k) m = IS_MAX ? max_skipping_nan<T>(m, x[u][k]) : min_skipping_nan<T>(m, x[u][k]);
            }
            // false for a NaN on either side, which sends the blocks on
            if (IS_MAX ? (m <= acc.value) : (m >= acc.value)) {
                if (is_float_t<T>::value || acc.index != kNone) return;
            }
            if (!is_float_t<T>::value || !isnan_t(m)) {
                // the group's extreme is a number: where it first occurs, without a branch
                // (positions ascend with u, then k), then one merge. The value is taken from
                // that position: of +0 and -0 the earlier counts.
                IDX first = (IDX)idx[0];
                T v = m;
#pragma unroll
                for (int u = U - 1; u >= 0; --u) {
#pragma unroll
                    for (int k = N - 1; k >= 0; --k) {
                        const bool hit = x[u][k] == m;
                        first = hit ? (IDX)(idx[u] + k) : first;
                        v = hit ? x[u][k] : v;
                    }
                }
                combine(Acc{v, first}, acc);
                return;
            }
            // every element a NaN, or a signalling NaN poisoned m: the exact rule, block by block
        }
#pragma unroll
        for (int u = 0; u < U; ++u) accumulate_n<N>(x[u], idx[u], acc);
    }
    __device__ __forceinline__ void store(const Acc& acc, char* out, char*) const {
        if (out_mode == 0) *reinterpret_cast<T*>(out) = acc.value;
        else if (out_mode == 4) *reinterpret_cast<int32_t*>(out) = (int32_t)acc.index;
        else *reinterpret_cast<int64_t*>(out) = (int64_t)acc.index;
    }
};

// ---- min / max, value only ---------------------------------------------------------
// The answer of min/max is a value, and an index is needed for it in one case only:
// when the extreme is a zero and zeros of both signs may be present, Numo's
// sequential loop keeps the one that came first (real_accum.h:217-278). So the
// fold keeps just the value, with the library's NaN-skipping max/min, and where it
// ends on a zero the kernels fold that output once more with the exact rule.
// An output that is all NaN stays NaN.
template <class T, bool IS_MAX>
struct ValueExtremeImpl {
    typedef T In;
    typedef T Acc;
    typedef ArgImpl<T, IS_MAX, false> Exact;
    static constexpr bool USES_INDEX = false;
    static constexpr int NOUT = 1;
    static constexpr bool HAS_EXACT = is_float_t<T>::value;
    // (rows first, then the rows' results: the zero that comes first in a row, then the row that comes first)
    static constexpr bool OWN_RESULTS = true;
    ValueExtremeImpl before_the_last() const { return *this; }
    static __device__ __forceinline__ float pick(float a, float b) { return IS_MAX ? __builtin_fmaxf(a, b) : __builtin_fminf(a, b); }
    static __device__ __forceinline__ double pick(double a, double b) { return IS_MAX ? __builtin_fmax(a, b) : __builtin_fmin(a, b); }
    static __device__ __forceinline__ int32_t pick(int32_t a, int32_t b) { return IS_MAX ? (a > b ? a : b) : (a < b ? a : b); }
    __device__ __forceinline__ Acc identity() const {
        if (is_float_t<T>::value) return Lim<T>::skip();
        return IS_MAX ? Lim<T>::lowest() : Lim<T>::highest();
    }
    __device__ __forceinline__ void combine(const Acc& next, Acc& acc) const { acc = pick(acc, next); }
    __device__ __forceinline__ void accumulate(T x, int64_t, Acc& acc) const { acc = pick(acc, x); }
    template <int N>
    __device__ __forceinline__ void accumulate_n(const T (&x)[N], int64_t, Acc& acc) const {
#pragma unroll
        for (int k = 0; k < N; ++k) acc = pick(acc, x[k]);
    }
    // a whole step at once (no test per vector between the loads' arrivals)
    static constexpr bool GROUPED = true;
    template <int U, int N>
    __device__ __forceinline__ void accumulate_group(const T (&x)[U][N], const int64_t (&)[U], Acc& acc) const {
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int k = 0; k < N; ++k) acc = pick(acc, x[u][k]);
        }
    }
    __device__ __forceinline__ bool needs_exact(const Acc& acc) const { return acc == (T)0; }
    __host__ __device__ __forceinline__ Exact exact() const { return Exact{0}; }
    __device__ __forceinline__ Acc from_exact(const typename Exact::Acc& e) const { return e.value; }
    __device__ __forceinline__ void store(const Acc& acc, char* out, char*) const { *reinterpret_cast<T*>(out) = acc; }
};

// ---- minmax / ptp ------------------------------------------------------------------
// Both ends at once, each with its index so that minmax answers exactly what min
// and max answer (real_accum_kernel.cu:54-84,139-157).
// out_mode: 0 = two outputs (minmax), 1 = max - min (ptp).
template <class T, bool NAN_WINS>
struct MinMaxImpl {
    typedef T In;
    typedef typename ArgImpl<T, false, NAN_WINS>::Acc One;
    struct Acc { One lo; One hi; };
    static constexpr bool USES_INDEX = true;
    static constexpr int NOUT = 2;
    int out_mode;
    __device__ __forceinline__ Acc identity() const {
        ArgImpl<T, false, NAN_WINS> a{0};
        ArgImpl<T, true, NAN_WINS> b{0};
        const typename ArgImpl<T, true, NAN_WINS>::Acc h = b.identity();
        return Acc{a.identity(), One{h.value, h.index}};
    }
    __device__ __forceinline__ void combine(const Acc& next, Acc& acc) const {
        ArgImpl<T, false, NAN_WINS> a{0};
        ArgImpl<T, true, NAN_WINS> b{0};
        a.combine(next.lo, acc.lo);
        typename ArgImpl<T, true, NAN_WINS>::Acc h{acc.hi.value, acc.hi.index};
        b.combine(typename ArgImpl<T, true, NAN_WINS>::Acc{next.hi.value, next.hi.index}, h);
        acc.hi = One{h.value, h.index};
    }
    __device__ __forceinline__ void accumulate(T x, int64_t idx, Acc& acc) const { combine(Acc{One{x, idx}, One{x, idx}}, acc); }
    // (an accumulator {lo, hi} of the value-only form this is the exact rule of, folded as one element per end at position idx)
    template <class P>
    __device__ __forceinline__ void accumulate_acc(const P& part, int64_t idx, Acc& acc) const {
        combine(Acc{One{part.lo, idx}, One{part.hi, idx}}, acc);
    }
    template <int N>
    __device__ __forceinline__ void accumulate_n(const T (&x)[N], int64_t idx0, Acc& acc) const {
        // each end runs its own block rule
        ArgImpl<T, false, NAN_WINS> a{0};
        ArgImpl<T, true, NAN_WINS> b{0};
        a.template accumulate_n<N>(x, idx0, acc.lo);
        typename ArgImpl<T, true, NAN_WINS>::Acc h{acc.hi.value, acc.hi.index};
        b.template accumulate_n<N>(x, idx0, h);
        acc.hi = One{h.value, h.index};
    }
    // a whole step at once: each end runs its own group rule (one comparison when nothing in the
    // step can change that end)
    static constexpr bool GROUPED = true;
    template <int U, int N>
    __device__ __forceinline__ void accumulate_group(const T (&x)[U][N], const int64_t (&idx)[U], Acc& acc) const {
        ArgImpl<T, false, NAN_WINS> a{0};
        ArgImpl<T, true, NAN_WINS> b{0};
        a.template accumulate_group<U, N>(x, idx, acc.lo);
        typename ArgImpl<T, true, NAN_WINS>::Acc h{acc.hi.value, acc.hi.index};
        b.template accumulate_group<U, N>(x, idx, h);
        acc.hi = One{h.value, h.index};
    }
    __device__ __forceinline__ void store(const Acc& acc, char* out, char* out2) const {
        if (out_mode == 0) {
            *reinterpret_cast<T*>(out) = acc.lo.value;
            *reinterpret_cast<T*>(out2) = acc.hi.value;
        } else {
            // (+0) - (-0) and the like: Numo keeps one element for both ends, so a
            // zero spread is +0 (types/real_accum.h:406-441)
            T d = spread<T>(acc.hi.value, acc.lo.value);
            if (d == (T)0) d = (T)0;
            *reinterpret_cast<T*>(out) = d;
        }
    }
};

// Both ends by value alone, for the answers that do not depend on which of two equal elements came
// first: ptp always (a zero's sign drops out of hi - lo, and a zero spread is +0 by rule), minmax of
// integers (equal integers are the same answer). One min and one max per element, no index carried
// through the fold: the index-carrying form above costs a third of the memory rate on large arrays.
// NaN is skipped unless an output holds nothing else (the rule without `nan: true`).
// out_mode: 0 = two outputs (minmax), 1 = max - min (ptp).
template <class T, bool EXACT_ZEROS = false>
struct MinMaxValueImpl {
    typedef T In;
    struct Acc { T lo; T hi; };
    static constexpr bool USES_INDEX = false;
    static constexpr int NOUT = 2;
    // EXACT_ZEROS (float minmax): an end that comes out as a zero may be +0 or -0 depending on which came first;
    // the kernels that know this protocol then go over the output again with the index-carrying rule
    typedef MinMaxImpl<T, false> Exact;
    static constexpr bool HAS_EXACT = EXACT_ZEROS && is_float_t<T>::value;
    int out_mode;
    __device__ __forceinline__ bool needs_exact(const Acc& acc) const { return acc.lo == (T)0 || acc.hi == (T)0; }
    __host__ __device__ __forceinline__ Exact exact() const { return Exact{out_mode}; }
    __device__ __forceinline__ Acc from_exact(const typename Exact::Acc& e) const { return Acc{e.lo.value, e.hi.value}; }
    // (the library's fmin / fmax: of a number and a NaN the number, a signalling NaN included)
    static __device__ __forceinline__ float lower(float a, float b) { return __builtin_fminf(a, b); }
    static __device__ __forceinline__ double lower(double a, double b) { return __builtin_fmin(a, b); }
    static __device__ __forceinline__ int32_t lower(int32_t a, int32_t b) { return a < b ? a : b; }
    static __device__ __forceinline__ float upper(float a, float b) { return __builtin_fmaxf(a, b); }
    static __device__ __forceinline__ double upper(double a, double b) { return __builtin_fmax(a, b); }
    static __device__ __forceinline__ int32_t upper(int32_t a, int32_t b) { return a > b ? a : b; }
    __device__ __forceinline__ Acc identity() const {
        if (is_float_t<T>::value) return Acc{Lim<T>::skip(), Lim<T>::skip()};
        return Acc{Lim<T>::highest(), Lim<T>::lowest()};
    }
    __device__ __forceinline__ void combine(const Acc& next, Acc& acc) const {
        acc.lo = lower(acc.lo, next.lo);
        acc.hi = upper(acc.hi, next.hi);
    }
    __device__ __forceinline__ void accumulate(T x, int64_t, Acc& acc) const {
        acc.lo = lower(acc.lo, x);
        acc.hi = upper(acc.hi, x);
    }
    template <int N>
    __device__ __forceinline__ void accumulate_n(const T (&x)[N], int64_t, Acc& acc) const {
#pragma unroll
        for (int k = 0; k < N; ++k) {
            acc.lo = lower(acc.lo, x[k]);
            acc.hi = upper(acc.hi, x[k]);
        }
    }
    static constexpr bool GROUPED = true;
    template <int U, int N>
    __device__ __forceinline__ void accumulate_group(const T (&x)[U][N], const int64_t (&)[U], Acc& acc) const {
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int k = 0; k < N; ++k) {
                acc.lo = lower(acc.lo, x[u][k]);
                acc.hi = upper(acc.hi, x[u][k]);
            }
        }
    }
    __device__ __forceinline__ void store(const Acc& acc, char* out, char* out2) const {
        if (out_mode == 0) {
            *reinterpret_cast<T*>(out) = acc.lo;
            *reinterpret_cast<T*>(out2) = acc.hi;
        } else {
            T d = spread<T>(acc.hi, acc.lo);
            if (d == (T)0) d = (T)0;  // (+0) - (-0) and the like: +0 (types/real_accum.h:406-441)
            *reinterpret_cast<T*>(out) = d;
        }
    }
};

}  // namespace cumo_hip

#endif