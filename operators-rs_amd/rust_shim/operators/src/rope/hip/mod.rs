//! rope on the MI355X backend (`ophip_rope_*`).  The kernel computes sin / cos itself, so the
//! table `build_sincos` returns is empty, as the CPU and CUDA backends' is.
use super::{fill_pos, Args, Rope, Seq, SinCosTable};
use crate::hip::{ffi, hip_operator, layout_of, upload};
use digit_layout::{types as ty, DigitLayout};

hip_operator! {
    Rope, ffi::ophip_rope, ffi::ophip_rope_args,
    ophip_rope_create, ophip_rope_scheme, ophip_rope_launch, ophip_rope_destroy,
    |a| ffi::ophip_rope_args {
        t_layout: layout_of(&a.t_layout),
        t_base: a.t_base.cast(),
        p_layout: layout_of(&a.p_layout),
        p_base: a.p_base.cast(),
        sin_layout: layout_of(&a.sin_layout),
        sin_base: a.sin_base.cast(),
        cos_layout: layout_of(&a.cos_layout),
        cos_base: a.cos_base.cast(),
        theta: a.theta,
    };

    fn build_sincos<QA>(_dt: DigitLayout, _nctx: usize, _dh: usize, queue_alloc: &QA) -> SinCosTable<QA::DevMem>
    where
        QA: crate::QueueAlloc<Hardware = Self::Hardware>,
    {
        SinCosTable {
            nctx: 0,
            mem: queue_alloc.alloc(0),
        }
    }

    fn build_pos<I, QA>(dt: DigitLayout, nt: usize, iter: I, queue_alloc: &QA) -> QA::DevMem
    where
        I: IntoIterator<Item = Seq>,
        QA: crate::QueueAlloc<Hardware = Self::Hardware>,
    {
        let mut host = vec![0u64; (nt * dt.nbytes()).div_ceil(8)];
        match dt {
            ty::U32 => fill_pos(host.as_mut_ptr().cast::<u32>(), nt, iter),
            ty::U64 => fill_pos(host.as_mut_ptr(), nt, iter),
            _ => todo!(),
        }
        let bytes = unsafe { std::slice::from_raw_parts(host.as_ptr().cast::<u8>(), nt * dt.nbytes()) };
        upload(bytes, queue_alloc)
    }
}
