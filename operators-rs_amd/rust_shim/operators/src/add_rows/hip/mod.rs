//! add_rows on the MI355X backend (`ophip_add_rows_*`): dst[b, m, :] += src[idx[b, m], :].
use super::{AddRows, Args};
use crate::hip::{ffi, hip_operator, layout_of};

hip_operator! {
    AddRows, ffi::ophip_add_rows, ffi::ophip_add_rows_args,
    ophip_add_rows_create, ophip_add_rows_scheme, ophip_add_rows_launch, ophip_add_rows_destroy,
    |a| ffi::ophip_add_rows_args {
        dst_layout: layout_of(&a.dst_layout),
        dst_base: a.dst_base.cast(),
        src_layout: layout_of(&a.src_layout),
        src_base: a.src_base.cast(),
        idx_layout: layout_of(&a.idx_layout),
        idx_base: a.idx_base.cast(),
    };
}
