//! layer_norm on the MI355X backend (`ophip_layer_norm_*`).
use super::{Args, LayerNorm};
use crate::hip::{ffi, hip_operator, layout_of};

hip_operator! {
    LayerNorm, ffi::ophip_layer_norm, ffi::ophip_layer_norm_args,
    ophip_layer_norm_create, ophip_layer_norm_scheme, ophip_layer_norm_launch, ophip_layer_norm_destroy,
    |a| ffi::ophip_layer_norm_args {
        y_layout: layout_of(&a.y_layout),
        y_base: a.y_base.cast(),
        x_layout: layout_of(&a.x_layout),
        x_base: a.x_base.cast(),
        scale_layout: layout_of(&a.scale_layout),
        scale_base: a.scale_base.cast(),
        bias_layout: layout_of(&a.bias_layout),
        bias_base: a.bias_base.cast(),
        epsilon: a.epsilon,
    };
}
