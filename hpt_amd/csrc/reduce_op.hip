// One reduction op for all thirteen dtypes. Compiled once per op with
// -DHPT_REDUCE_ENTRY=<n> (see reduce_entry.hpp for the numbering).
#include "reduce_entry.hpp"
#include "reduce_kernels.hpp"

#ifndef HPT_REDUCE_ENTRY
#error "compile with -DHPT_REDUCE_ENTRY=<op number>"
#endif

namespace hpt {

namespace {

constexpr int E = HPT_REDUCE_ENTRY;

template <class T> struct OpFor {
    static constexpr bool arith = (E == HPT_SUM || E == HPT_PROD || E == HPT_NANSUM ||
                                   E == HPT_NANPROD || E == HPT_REDUCEL1 || E == HPT_SUM_SQUARE);
    static constexpr bool minmax = (E == HPT_MAX || E == HPT_MIN);
    static constexpr bool flt = (E == HPT_MEAN || E == HPT_REDUCEL2 || E == HPT_REDUCEL3 ||
                                 E == HPT_LOGSUMEXP);
    static constexpr bool boolean = (E == HPT_ALL || E == HPT_ANY);
    using type = typename std::conditional<
        arith, ArithOp<E, T>,
        typename std::conditional<
            minmax, MinMaxOp<E, T>,
            typename std::conditional<
                flt, FloatOp<E, T>,
                typename std::conditional<boolean, BoolOp<E, T>,
                                          ArgOp<E == kArgMaxEntry, T>>::type>::type>::type>::type;
};

template <int DT> void launch_dt(const ReducePlan& p, const void* in, void* out,
                                 const ReduceScratch& sc, hipStream_t st, int init_out) {
    using T = typename DType<DT>::type;
    launch_reduce_t<typename OpFor<T>::type>(p, in, out, sc, st, init_out);
}

template <int DT> constexpr size_t acc_size_dt() {
    using T = typename DType<DT>::type;
    return sizeof(typename OpFor<T>::type::Acc);
}

const ReduceEntry kEntry = {
    {
#define X(DT) &launch_dt<DT>,
        HPT_FOR_ALL_DTYPES(X)
#undef X
    },
    {
#define X(DT) acc_size_dt<DT>(),
        HPT_FOR_ALL_DTYPES(X)
#undef X
    }};

}  // namespace

template <> const ReduceEntry& reduce_entry<HPT_REDUCE_ENTRY>() { return kEntry; }

}  // namespace hpt
