//! random_sample on the MI355X backend (`ophip_random_sample_*`).  The kernels take candidate
//! indices from positions, so `indices` is validated but never read; `build_indices` still fills it
//! for callers that share one `Args` between backends.
use super::{Args, Indices, RandomSample};
use crate::hip::{ffi, hip_operator, layout_of, upload};

hip_operator! {
    RandomSample, ffi::ophip_random_sample, ffi::ophip_random_sample_args,
    ophip_random_sample_create, ophip_random_sample_scheme, ophip_random_sample_launch, ophip_random_sample_destroy,
    |a| ffi::ophip_random_sample_args {
        kv_pair: layout_of(&a.kv_pair),
        kv_pair_base: a.kv_pair_base.cast(),
        logits: layout_of(&a.logits),
        logits_base: a.logits_base.cast(),
        indices: layout_of(&a.indices),
        indices_base: a.indices_base.cast(),
        config: ffi::ophip_sample_args {
            temperature: a.config.temperature,
            top_p: a.config.top_p,
            top_k: a.config.top_k,
        },
        seed: a.seed,
    };

    fn build_indices<QA>(n: usize, queue_alloc: &QA) -> Indices<QA::DevMem>
    where
        QA: crate::QueueAlloc<Hardware = Self::Hardware>,
    {
        let host = (0..n as u32).collect::<Vec<_>>();
        let bytes = unsafe { std::slice::from_raw_parts(host.as_ptr().cast::<u8>(), n * 4) };
        Indices {
            n,
            mem: upload(bytes, queue_alloc),
        }
    }
}
