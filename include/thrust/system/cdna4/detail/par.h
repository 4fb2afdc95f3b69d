// thrust::system::cdna4::detail::par_t, par_nosync_t, execute_on_stream and the objects par /
// par_nosync (the counterpart of thrust/system/cuda/detail/par.h:44-238); defined with the
// system's core in core.h.
#pragma once
#include <thrust/system/cdna4/detail/core.h>
