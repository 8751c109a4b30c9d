"""verinf_amd -- MI355X (gfx950) kernels for the VerInf prover's Goldilocks hot path.

Layout mirrors the reference modules this package stands in for:

    verinf_amd.prover.cuda_primitives   field ops, NTT, coset LDE   (prover/cuda_primitives.py)
    verinf_amd.prover.kquant_cuda       K-quant blocks -> field     (prover/kquant_cuda.py)
    verinf_amd.prover.protocol          field / domain definitions  (prover/protocol.py, pure maths part)
    verinf_amd.layergkr.gpu             encode_batch_ntt, fold_t, gl_sum, prove_terms_gpu (layergkr/gpu.py)
    verinf_amd.layergkr.rs              Commit.from_messages / encode gates (layergkr/rs.py)
    verinf_amd.layergkr.sumcheck        prove / prove_terms / verify (layergkr/sumcheck.py)

Everything computes through libverinf_hip.so (hand-written HIP, C ABI in
include/verinf_hip.h); there is no CPU fallback.
"""
__version__ = "0.2"
