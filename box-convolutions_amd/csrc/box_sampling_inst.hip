// Explicit instantiations of the box-sampling launch templates (box_sampling_impl.hpp). This file
// is compiled several times: BOXCONV_INST_T / BOXCONV_INST_TG select the arithmetic type and the
// element type of grad_output / grad_input, BOXCONV_INST_PART the half of the templates
//   1: the streaming pass over grad_output
//   2: the gradient w.r.t. the input, and (where T == TG) the gather and finalize launches.
//   3: (T = float) the streaming pass's variant with consecutive columns per lane;
//   4: the same variant for the parameter sums alone.

#include "box_sampling_impl.hpp"

namespace boxconv {

#if BOXCONV_INST_PART == 1
template hipError_t grad_output_stream_launch<BOXCONV_INST_T, BOXCONV_INST_TG>(
    const BOXCONV_INST_T*, const BOXCONV_INST_TG*, BoxParams<BOXCONV_INST_T>, double*, int, BOXCONV_INST_T*,
    const StreamPlan&, Dims, bool, hipStream_t);
#elif BOXCONV_INST_PART == 3
template hipError_t grad_output_stream_consec_launch<BOXCONV_INST_TG, true>(const SampleArgs<float>&, int, int, bool,
                                                                            dim3, hipStream_t);
#elif BOXCONV_INST_PART == 4
template hipError_t grad_output_stream_consec_launch<BOXCONV_INST_TG, false>(const SampleArgs<float>&, int, int, bool,
                                                                             dim3, hipStream_t);
#else
template hipError_t grad_input_launch<BOXCONV_INST_T, BOXCONV_INST_TG>(
    const BOXCONV_INST_T*, int, BoxParams<BOXCONV_INST_T>, BOXCONV_INST_TG*, Dims, bool, bool, hipStream_t,
    const ParamFinish<BOXCONV_INST_T>*, bool*);
#ifdef BOXCONV_INST_SAME_TYPE
template hipError_t grad_params_gather_launch<BOXCONV_INST_T>(const BOXCONV_INST_T*, const BOXCONV_INST_T*,
                                                              BoxParams<BOXCONV_INST_T>, double*, Dims, bool,
                                                              hipStream_t);
template hipError_t grad_params_finish<BOXCONV_INST_T>(const ParamFinish<BOXCONV_INST_T>&,
                                                       BoxParams<BOXCONV_INST_T>, hipStream_t);
#endif
#endif

}  // namespace boxconv
