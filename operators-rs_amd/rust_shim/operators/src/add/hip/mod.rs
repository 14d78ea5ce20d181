//! add on the MI355X backend (`ophip_add_*`): c = a + b, any strides (0 broadcasts a or b).
use super::{Add, Args};
use crate::hip::{ffi, hip_operator, layout_of};

hip_operator! {
    Add, ffi::ophip_add, ffi::ophip_add_args,
    ophip_add_create, ophip_add_scheme, ophip_add_launch, ophip_add_destroy,
    |a| ffi::ophip_add_args {
        c_layout: layout_of(&a.c_layout),
        c_base: a.c_base.cast(),
        a_layout: layout_of(&a.a_layout),
        a_base: a.a_base.cast(),
        b_layout: layout_of(&a.b_layout),
        b_base: a.b_base.cast(),
    };
}
