//! gelu on the MI355X backend (`ophip_gelu_*`), in place, tanh form.
use super::{Args, Gelu};
use crate::hip::{ffi, hip_operator, layout_of};

hip_operator! {
    Gelu, ffi::ophip_gelu, ffi::ophip_gelu_args,
    ophip_gelu_create, ophip_gelu_scheme, ophip_gelu_launch, ophip_gelu_destroy,
    |a| ffi::ophip_gelu_args {
        layout: layout_of(&a.layout),
        base: a.base.cast(),
    };
}
