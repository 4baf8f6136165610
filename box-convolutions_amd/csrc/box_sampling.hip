// Host-side pieces of the box-sampling kernels that do not depend on the element type; the
// kernels themselves are templates in box_sampling_impl.hpp, instantiated by box_sampling_inst.hip.

#include "box_sampling_impl.hpp"   // stream_lds_bytes; the templates in it are not instantiated here

namespace boxconv {

bool force_gather_kernels() {
    const char* e = std::getenv("BOXCONV_FORCE_GATHER");
    return e != nullptr && e[0] == '1';
}

namespace {

__global__ void fill_zero_kernel(double* __restrict__ p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.0;
}

}  // namespace

hipError_t grad_params_begin(double* acc, int n_boxes, hipStream_t stream) {
    if (n_boxes == 0) return hipSuccess;
    BOXCONV_LAUNCH("fill_zero", fill_zero_kernel, dim3((n_boxes * 5 + 255) / 256), dim3(256), 0,
                   stream, acc, n_boxes * 5);
    return hipGetLastError();
}

StreamPlan plan_grad_output_stream(int64_t planes_f, int h, int w, size_t elem_size) {
    StreamPlan sp{};
    const RowConfig rc = stream_row_config(std::max(w, 1));
    sp.usable = row_kernels_apply(h, w, elem_size) &&
                stream_lds_bytes(rc.K, rc.nt, elem_size) <= kMaxDynamicLds;
    int nb = bands_for(std::max<int64_t>(planes_f, 1), h, 32, 2048);
    int R = (h + nb - 1) / nb;
    R += R & 1;                                        // rows are handled in pairs
    sp.R = std::max(R, 2);
    sp.nb = (h + sp.R - 1) / sp.R;
    sp.parts = rc.nt == 1024 ? 2 : 1;
    return sp;
}

}  // namespace boxconv
