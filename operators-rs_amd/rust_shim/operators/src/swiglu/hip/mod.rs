//! swiglu on the MI355X backend (`ophip_swiglu_*`).
use super::{Args, Swiglu};
use crate::hip::{ffi, hip_operator, layout_of};

hip_operator! {
    Swiglu, ffi::ophip_swiglu, ffi::ophip_swiglu_args,
    ophip_swiglu_create, ophip_swiglu_scheme, ophip_swiglu_launch, ophip_swiglu_destroy,
    |a| ffi::ophip_swiglu_args {
        gate_layout: layout_of(&a.gate_layout),
        gate_base: a.gate_base.cast(),
        up_layout: layout_of(&a.up_layout),
        up_base: a.up_base.cast(),
    };
}
