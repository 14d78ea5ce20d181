//! fuesd_softmax on the MI355X backend (`ophip_fused_softmax_*`).
use super::{Args, FusedSoftmax};
use crate::hip::{ffi, hip_operator, layout_of};

hip_operator! {
    FusedSoftmax, ffi::ophip_fused_softmax, ffi::ophip_fused_softmax_args,
    ophip_fused_softmax_create, ophip_fused_softmax_scheme, ophip_fused_softmax_launch, ophip_fused_softmax_destroy,
    |a| ffi::ophip_fused_softmax_args {
        att_mask: a.att_mask as u8, // AttnMask is repr(u8): None = 0, Causal = 1
        att_layout: layout_of(&a.att_layout),
        att_base: a.att_base.cast(),
    };
}
