// Umbrella header of the ark:: API served by the MI355X backend.
#ifndef ARK_HPP
#define ARK_HPP

#include <ark/context.hpp>
#include <ark/data_type.hpp>
#include <ark/dims.hpp>
#include <ark/error.hpp>
#include <ark/executor.hpp>
#include <ark/init.hpp>
#include <ark/log.hpp>
#include <ark/model.hpp>
#include <ark/model_ref.hpp>
#include <ark/planner.hpp>
#include <ark/random.hpp>
#include <ark/tensor.hpp>
#include <ark/version.hpp>

#endif  // ARK_HPP
