// Runs the fused-attention kernels (daceml_amd/csrc/attention.hip, compiled for the host against emu.h) on one
// problem. TEST INFRASTRUCTURE ONLY; built and driven by tests/test_kernel_emulation.py.
#include <stdarg.h>
#include <stdio.h>

#include "attention_emu.h"

namespace dml {
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vfprintf(stderr, fmt, ap);
    va_end(ap);
    fputc('\n', stderr);
}
int launch_status(const char*) { return 0; }

namespace {

alignas(16) char lds[160 * 1024];

struct Call {
    const _Float16 *q, *k, *v, *o, *d_o;
    _Float16 *out, *dq, *dk, *dv;
    float *lse, *dvec;
    AttnArgs a;
    AttnArgsMasked m;
};

template <bool MASK> const AttnArgsFor<MASK>& args_of(const Call* c);
template <> const AttnArgs& args_of<false>(const Call* c) { return c->a; }
template <> const AttnArgsMasked& args_of<true>(const Call* c) { return c->m; }

template <bool MASK> void fwd(void* p) {
    const Call* c = static_cast<const Call*>(p);
    attention_fwd_kernel<MASK>(c->q, c->k, c->v, c->out, c->lse, args_of<MASK>(c));
}
template <bool MASK> void bwd_dq(void* p) {
    const Call* c = static_cast<const Call*>(p);
    attention_bwd_dq_kernel<MASK>(c->q, c->k, c->v, c->o, c->lse, c->d_o, c->dq, c->dvec, args_of<MASK>(c));
}
template <bool MASK> void bwd_dkv(void* p) {
    const Call* c = static_cast<const Call*>(p);
    attention_bwd_dkv_kernel<MASK>(c->q, c->k, c->v, c->lse, c->dvec, c->d_o, c->dk, c->dv, args_of<MASK>(c));
}

}  // namespace
}  // namespace dml

using namespace dml;

// which: 0 forward (writes out, lse), 1 the dQ kernel (reads out as O, lse; writes dq and the row dots dvec), 2 the
// dK / dV kernel (reads lse, dvec; writes dk, dv). All tensors dense [b0, b1, seq, 64]; mask NULL or fp16 rows with
// the two batch strides in mask_stride. Returns 0, 1 on a deadlock, negative for rejected arguments.
extern "C" int emu_attention(int which, const dmlhip_attention_desc* d, const void* q, const void* k, const void* v,
                             void* out, float* lse, const void* d_o, void* dq, void* dk, void* dv, float* dvec,
                             const void* mask, const int64_t* mask_stride, unsigned seed, int late_dma) {
    Call c = {};
    if (int e = fill_args(d, d, c.a, "emu_attention")) return e;
    c.q = (const _Float16*)q; c.k = (const _Float16*)k; c.v = (const _Float16*)v;
    c.out = (_Float16*)out; c.o = (const _Float16*)out; c.lse = lse; c.d_o = (const _Float16*)d_o;
    c.dq = (_Float16*)dq; c.dk = (_Float16*)dk; c.dv = (_Float16*)dv; c.dvec = dvec;
    const long long bh = (long long)d->batch[0] * d->batch[1];
    const long long blocks = which == 2 ? bh * ((c.a.seq_k + 127) / 128) : bh * c.a.q_tiles;
    c.a.total_blocks = blocks;
    if (mask)
        if (int e = fill_mask(c.a, mask, mask_stride, c.m, "emu_attention")) return e;
    emu::kernel_fn fn = which == 0 ? (mask ? fwd<true> : fwd<false>)
                      : which == 1 ? (mask ? bwd_dq<true> : bwd_dq<false>) : (mask ? bwd_dkv<true> : bwd_dkv<false>);
    return emu::run_grid(fn, &c, (unsigned)blocks, kAttnThreads, seed, late_dma, lds);
}
