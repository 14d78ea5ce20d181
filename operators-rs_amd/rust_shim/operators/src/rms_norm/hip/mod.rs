//! rms_norm on the MI355X backend (`ophip_rms_norm_*`).
use super::{Args, RmsNorm};
use crate::hip::{ffi, hip_operator, layout_of};

hip_operator! {
    RmsNorm, ffi::ophip_rms_norm, ffi::ophip_rms_norm_args,
    ophip_rms_norm_create, ophip_rms_norm_scheme, ophip_rms_norm_launch, ophip_rms_norm_destroy,
    |a| ffi::ophip_rms_norm_args {
        y_layout: layout_of(&a.y_layout),
        y_base: a.y_base.cast(),
        x_layout: layout_of(&a.x_layout),
        x_base: a.x_base.cast(),
        w_layout: layout_of(&a.w_layout),
        w_base: a.w_base.cast(),
        epsilon: a.epsilon,
    };
}
