//! rearrange on the MI355X backend (`ophip_rearrange_*`): any rank up to 8 merged dimensions,
//! any unit size, negative and zero source strides.
use super::{Args, Rearrange};
use crate::hip::{ffi, hip_operator, layout_of};

hip_operator! {
    Rearrange, ffi::ophip_rearrange, ffi::ophip_rearrange_args,
    ophip_rearrange_create, ophip_rearrange_scheme, ophip_rearrange_launch, ophip_rearrange_destroy,
    |a| ffi::ophip_rearrange_args {
        dst_layout: layout_of(&a.dst_layout),
        dst_base: a.dst_base.cast(),
        src_layout: layout_of(&a.src_layout),
        src_base: a.src_base.cast(),
    };
}
