// Finite-p forward on images: the tiled kernels extract the patches of the convolutional layer while they load their
// tiles, so the unfolded tensor [B, C*kh*kw, OH*OW] that the reference materialises (core/modules/norm_dist.py:93-102)
// is never written or read.  Same operator policies as the fully-connected forward; the plain kernels only (the
// seeded and probed variants of the large exponents need k contiguous).
#include "fwd_norm_ops.h"

namespace ndist {

template <int IP>
static int launch_sum_conv(const FwdParams& P, hipStream_t st) {
    return launch_fwd_conv<OpSum<IP>, CfgWide4, CfgBig, CfgSmall>(P, st);
}

int launch_norm_forward_conv(const float* x, const float* w, const Geom& s, float* out, float p, hipStream_t st,
                             const UnfoldGeom& cv) {
    FwdParams P{};
    P.x = x;
    P.w = w;
    P.out = out;
    P.s = s;
    P.p = p;
    P.inv_p = 1.0f / p;
    P.implicit = 1;
    P.pm = make_patch_map(cv, s.G);
    if (p > kMinNormalizedP) return launch_fwd_conv<OpNormalized<false>, CfgWideT, CfgMid, CfgSmall>(P, st);
    if (p == (float)(int)p) {
        switch ((int)p) {
            case 1: return launch_sum_conv<1>(P, st);
            case 2: return launch_sum_conv<2>(P, st);
            case 3: return launch_sum_conv<3>(P, st);
            case 4: return launch_sum_conv<4>(P, st);
            case 5: return launch_sum_conv<5>(P, st);
            case 6: return launch_sum_conv<6>(P, st);
            case 7: return launch_sum_conv<7>(P, st);
            case 8: return launch_sum_conv<8>(P, st);
            case 9: return launch_sum_conv<9>(P, st);
            case 10: return launch_sum_conv<10>(P, st);
            default: break;
        }
    }
    return launch_sum_conv<0>(P, st);
}

}  // namespace ndist
