// double instantiation of every kernel launcher.
#include "sb_launch_impl.hpp"

namespace sb {
SB_INSTANTIATE_LAUNCHERS(double)
}  // namespace sb
