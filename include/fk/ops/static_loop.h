// StaticLoop<Operation, ITERATIONS>: one Binary operation applied ITERATIONS times with the same parameters, unrolled at
// compile time.  Counterpart of the reference's algorithms/basic_ops/static_loop.h:21-45, including what it does for
// ITERATIONS <= 1: the operation is applied once.
#ifndef FK_OPS_STATIC_LOOP_H
#define FK_OPS_STATIC_LOOP_H

#include "fk/ops/arithmetic.h"

namespace fk {

template <typename Operation, int ITERATIONS>
struct StaticLoop {
private:
    using SelfType = StaticLoop<Operation, ITERATIONS>;
    template <int DONE>
    FK_HD_STATIC typename Operation::OutputType rest(const typename Operation::InputType& input, const typename Operation::ParamsType& params) {
        if constexpr (DONE < ITERATIONS) {
            return rest<DONE + 1>(Operation::exec(input, params), params);
        } else {
            return input;
        }
    }

public:
    FK_BINARY_OPERATION(StaticLoop, typename Operation::InputType, typename Operation::ParamsType, typename Operation::OutputType)
    static_assert(std::is_same_v<typename Operation::InputType, typename Operation::OutputType>, "the looped operation must map its type to itself");
    FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) { return rest<1>(Operation::exec(input, params), params); }
};

} // namespace fk
#endif
