// hmr_copy: strided copy with dtype conversion (ref: csrc/homura_rocm.h:138, csrc/copy.hip:131-151).
#include "ew_common.hpp"

extern "C" hmr_status hmr_copy(hmr_context_t ctx, const hmr_tensor_desc *dst, const hmr_tensor_desc *src) {
    return hmr::fenced([&] {
        const hmr_tensor_desc *descs[2] = {dst, src};
        return hmr::run_map(ctx, "copy", 2, descs, nullptr, [&](const hmr::MapCall &call, hipStream_t stream) {
            if (dst->dtype == src->dtype) {
                return hmr::with_word(hmr::dtype_size(dst->dtype), [&](auto w) {
                    hmr::launch_map<hmr::Move<typename decltype(w)::type>>(call, stream);
                });
            }
            bool done = false;
            hmr::with_any_type(src->dtype, [&](auto s) {
                using S = typename decltype(s)::type;
                done = hmr::with_any_type(dst->dtype, [&](auto d) {
                    using D = typename decltype(d)::type;
                    if constexpr (!std::is_same_v<D, S>) hmr::launch_map<hmr::Convert<D, S>>(call, stream);
                });
            });
            return done;
        });
    });
}
