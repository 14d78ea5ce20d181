//! mat_mul on the MI355X backend (`ophip_mat_mul_*`): MFMA kernels chosen per shape inside the
//! library.  Scalars follow the CPU backend (alpha and beta rounded to f16 for f16 data, C not
//! read when beta == 0).  `scheme` never fails, like the CUDA backend's: the attention
//! composites hand it layouts that are not yet a valid product.
use super::{Args, MatMul};
use crate::hip::{ffi, hip_operator, layout_of};

hip_operator! {
    MatMul, ffi::ophip_mat_mul, ffi::ophip_mat_mul_args,
    ophip_mat_mul_create, ophip_mat_mul_scheme, ophip_mat_mul_launch, ophip_mat_mul_destroy,
    |a| ffi::ophip_mat_mul_args {
        c_layout: layout_of(&a.c_layout),
        c_base: a.c_base.cast(),
        beta: a.beta,
        a_layout: layout_of(&a.a_layout),
        a_base: a.a_base.cast(),
        b_layout: layout_of(&a.b_layout),
        b_base: a.b_base.cast(),
        alpha: a.alpha,
    };
}
