// One whole optimiser step of a model group, issued from native code.
//
// A step on a small minibatch is eight to ten launches of 2-50 us each, so its cost is what the host
// spends per launch. Issued from here that is ~2.6 us per launch (measured on MI355X); from a scripting
// host, or as nodes of a multi-branch HIP graph, it is 6-8 us. The step is the body of the reference
// trainer's loop (deepity/deepity/sgd.py:98-135: gradstep with the batch gradient as its callback,
// deepity_smat.py:77-117), with the gradient computed by the fused kernels:
//
//   [P += mrate*mP]                                   Nesterov look-ahead       (gradstep.cu:41-51); kept in a vector
//                                                     of its own when the caller provides one, and then formed by
//                                                     the previous step's update kernel instead of a launch here
//   [Xd = input dropout(X)]                           dropoutord.py:50-70
//   pooled, argmax = scanpool_fprop(Wc, bc, Xd)       corr1ord -> bias -> relu -> poolrgn
//   Z, dpooled, dW1.. = head_train(pooled, Y)         dropout -> full (-> relu -> full) -> bias -> loss
//   dWc, dbc = scanpool_bprop(dpooled)
//   [dP += decay * sign(P)]                           L1 decay once it is switched on (full.py:111-119)
//   [dWc = 0]                                         scan filters still frozen
//   mP = mrate*mP - drate*dP ; P += ...               momentum / Nesterov update  (gradstep.cu:53-72)
//
// The same entry points a caller would use one by one are called in the same order, so the result is
// bit-identical to issuing them separately.
#include "dbk_common.h"
#include "scan_common.h"

namespace {

// The step's last kernel when the look-ahead lives beside the parameters: one pass over the flat vectors that
//   * adds up the partial results the backward kernels left (slabs of the scan filters' gradient as
//     reduce_slabs_kernel does, row chunks of the dense head's gradients as k_head_reduce does: same order),
//   * adds the L1 term, zeroes the scan filters' gradient while they are frozen, stores the gradient,
//   * applies the Nesterov update and forms the next step's look-ahead,
//   * writes the per-model loss when asked and moves the dropout generator on.
// (Sizes and offsets are 32-bit: the host checks that the flat vector and a slab have fewer than 2^31 elements. With
// 64-bit fields the kernel spilled a hundred scalar registers and divided 64-bit numbers per element.)
struct reduce_update_args {
    unsigned nparam;
    float *P, *L, *dP, *mP;
    const float *drate, *mrate, *decay;
    unsigned off_Wc, off_bc, off_W1, off_b1, off_W2, off_b2;
    unsigned nWc, nbc, nW1, nb1, nW2, nb2;
    const float* slabs; unsigned slab_stride; unsigned nslab;
    const float* head_partial; unsigned nchunk, pstride;
    unsigned nblock, k, h1, hidden;                                // k: rows of a model's block of W1
    int freeze_scan, loss_kind;
    float* loss; unsigned nrow;
    unsigned long long* counter; unsigned long long counter_advance;
};

__device__ __forceinline__ float chunk_sum(const reduce_update_args& a, unsigned b, unsigned idx)
{
    float s = 0.0f;
    for (unsigned c0 = 0; c0 < a.nchunk; c0 += 8) {                // eight chunks in flight per round, added in ascending order
        float v[8];
#pragma unroll
        for (unsigned t = 0; t < 8; ++t) v[t] = c0 + t < a.nchunk ? a.head_partial[((size_t)(c0 + t) * a.nblock + b) * a.pstride + idx] : 0.0f;
#pragma unroll
        for (unsigned t = 0; t < 8; ++t)
            if (c0 + t < a.nchunk) s += v[t];
    }
    return s;
}

// bx of gx: this workgroup's place among those that share the vector
__device__ __forceinline__ void reduce_update_body(const reduce_update_args& a, const unsigned bx, const unsigned gx)
{
    const unsigned nW1m = a.k * a.h1;                              // dense weights per model
    const unsigned total = a.nparam + (a.loss ? a.nblock : 0u);
    for (unsigned e = bx * blockDim.x + threadIdx.x; e < total; e += gx * blockDim.x) {
        if (e >= a.nparam) {                                       // per-model loss
            const unsigned b = (unsigned)(e - a.nparam);
            const float s = chunk_sum(a, b, nW1m + 2 * a.h1 + 1);
            a.loss[b] = dbk::loss_mean(a.loss_kind, s, (float)a.nrow);
            continue;
        }
        float g;
        bool scan_weight = false;
        if (e - a.off_Wc < a.nWc) { g = dbk_scan::slab_sum(a.slabs, a.slab_stride, e - a.off_Wc, a.nslab); scan_weight = true; }
        else if (e - a.off_bc < a.nbc) g = dbk_scan::slab_sum(a.slabs, a.slab_stride, a.nWc + (e - a.off_bc), a.nslab);
        else if (e - a.off_W1 < a.nW1) { const unsigned q = e - a.off_W1, b = q / nW1m; g = chunk_sum(a, b, q - b * nW1m); }
        else if (e - a.off_b1 < a.nb1) { const unsigned q = e - a.off_b1, b = q / a.h1; g = chunk_sum(a, b, nW1m + (q - b * a.h1)); }
        else if (e - a.off_W2 < a.nW2) { const unsigned q = e - a.off_W2, b = q / a.hidden; g = chunk_sum(a, b, nW1m + a.h1 + (q - b * a.hidden)); }
        else { const unsigned q = e - a.off_b2; g = chunk_sum(a, q, nW1m + 2 * a.h1); }
        const float look = a.L[e];
        if (a.decay) {
            const float sg = (float)((look > 0.0f) - (look < 0.0f));
            g += sg * a.decay[e];
        }
        if (scan_weight && a.freeze_scan) g = 0.0f;
        a.dP[e] = g;
        const float rm = a.mrate[e];
        const float delta = g * a.drate[e];
        const float mom = a.mP[e] * rm - delta;
        const float pn = look - delta;
        a.mP[e] = mom;
        a.P[e] = pn;
        a.L[e] = pn + rm * mom;
    }
    // every workgroup of the head kernel has read the generator position long ago: move it on
    if (a.counter && a.counter_advance && bx == 0 && threadIdx.x == 0) a.counter[0] += a.counter_advance;
}

__global__ __launch_bounds__(256) void k_reduce_update(reduce_update_args a) { reduce_update_body(a, blockIdx.x, gridDim.x); }

// The same for several model groups in one launch: workgroups first[g] .. first[g+1]-1 share group g's vector.
struct reduce_update_multi_args {
    unsigned n;
    unsigned first[dbk::MULTI_MAX + 1];
    reduce_update_args g[dbk::MULTI_MAX];
};
__global__ __launch_bounds__(256) void k_reduce_update_multi(const reduce_update_multi_args m)
{
    unsigned g = 0;
    while (g + 1 < m.n && blockIdx.x >= m.first[g + 1]) ++g;
    reduce_update_body(m.g[g], blockIdx.x - m.first[g], m.first[g + 1] - m.first[g]);
}

// Look-ahead vectors of several groups in one launch (L = P + mrate*mP, as k_lookahead forms it).
struct lookahead_multi_args {
    unsigned n;
    unsigned first[dbk::MULTI_MAX + 1];
    struct { size_t nparam; float* L; const float *P, *mP, *mrate; } g[dbk::MULTI_MAX];
};
__global__ __launch_bounds__(256) void k_lookahead_multi(const lookahead_multi_args m)
{
    unsigned g = 0;
    while (g + 1 < m.n && blockIdx.x >= m.first[g + 1]) ++g;
    const auto& a = m.g[g];
    const size_t gx = m.first[g + 1] - m.first[g];
    for (size_t e = (size_t)(blockIdx.x - m.first[g]) * blockDim.x + threadIdx.x; e < a.nparam; e += gx * blockDim.x)
        a.L[e] = a.P[e] + a.mrate[e] * a.mP[e];
}

__global__ void k_zero_f32(float* p, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0.0f;
}

}  // namespace

namespace {

// Sizes of a group's parameter blocks.
struct block_sizes { size_t F, k, kt, nWc, nW1, nb1, nW2, nb2; };
block_sizes sizes_of(const dbk_train_step_args* a)
{
    block_sizes z;
    z.F = a->nmodel * a->nfilter;                                  // filters of all models, side by side
    z.k = a->nfilter * (a->ptype == DBK_PT_ALL ? 2 : 1);           // pooled features per model
    z.nWc = 4 * a->m * z.F;
    z.kt = z.k + a->nfeat;                                         // rows of a model's block of W1: its inputs, then the shared feature columns
    z.nW1 = z.kt * a->nmodel * (a->hidden ? a->hidden : 1);
    z.nb1 = a->nmodel * (a->hidden ? a->hidden : 1);
    z.nW2 = a->hidden ? a->hidden * a->nmodel : 0;
    z.nb2 = a->hidden ? a->nmodel : 0;
    return z;
}

int check_args(const dbk_train_step_args* a)
{
    DBK_CHECK(a != nullptr, "ValueError: null argument block");
    DBK_CHECK(a->nmodel >= 1 && a->nfilter >= 1 && a->m >= 1, "ValueError: nmodel, nfilter and m must be >= 1");
    DBK_CHECK(a->ptype == DBK_PT_MAX || a->ptype == DBK_PT_AVG || a->ptype == DBK_PT_ALL,
              "ValueError: the fused step takes max, avg or all pooling");
    DBK_CHECK(a->P && a->dP && a->mP && a->drate && a->mrate, "ValueError: null parameter vector");
    DBK_CHECK(a->X && a->regions && a->Y && a->pooled && a->Z && a->dpooled, "ValueError: null batch or work buffer");
    DBK_CHECK(a->ptype == DBK_PT_AVG || a->argmax, "ValueError: max / all pooling needs the argmax work buffer");
    DBK_CHECK(a->input_rate <= 0.0f || (a->Xdrop && a->Mdrop), "ValueError: input dropout needs the Xdrop and Mdrop work buffers");
    DBK_CHECK(!(a->rate || a->input_rate > 0.0f) || a->counter, "ValueError: dropout needs the device generator position");
    const block_sizes z = sizes_of(a);
    const size_t need[6] = { a->off_Wc + z.nWc, a->off_bc + z.F, a->off_W1 + z.nW1, a->off_b1 + z.nb1,
                             a->off_W2 + z.nW2, a->off_b2 + z.nb2 };
    for (size_t v : need) DBK_CHECK(v <= a->nparam, "ValueError: a parameter block reaches past the flat vector (%zu > %zu)", v, a->nparam);
    return 0;
}

// Input dropout of one group (dropoutord.py:50-70): Xdrop = X with dropped letters, mirrored within (fwd, rev) pairs.
int drop_inputs(dbk_stream_t stream, const dbk_train_step_args* a)
{
    int rc = dbk_dropoutord_fp_tr(stream, a->X, a->Xdrop, a->Mdrop, a->N, a->input_rate, a->seed, 0, a->counter);
    if (rc) return rc;
    if (a->reverse_complement) {
        rc = dbk_dropoutord_mirror(stream, a->X, a->Xdrop, a->Mdrop, a->regions, a->nregion, a->m - 1);
        if (rc) return rc;
    }
    return dbk_counter_add(stream, a->counter, (a->N + 3) / 4);
}

// Arguments of the step's last kernel for one group, given where its partial sums lie.
int fill_update(reduce_update_args& u, const dbk_train_step_args* a, const block_sizes& z, const float* slabs, size_t slab_stride,
                unsigned nslab, const float* head_partial, unsigned nchunk, unsigned pstride, uint64_t draws)
{
    DBK_CHECK(a->nparam < ((size_t)1 << 31) && slab_stride < ((size_t)1 << 31) && a->nregion < ((size_t)1 << 31),
              "ValueError: a group's flat parameter vector is limited to 2^31 elements");
    u.nparam = (unsigned)a->nparam;
    u.P = a->P; u.L = a->L; u.dP = a->dP; u.mP = a->mP; u.drate = a->drate; u.mrate = a->mrate; u.decay = a->decay;
    u.off_Wc = (unsigned)a->off_Wc; u.off_bc = (unsigned)a->off_bc; u.off_W1 = (unsigned)a->off_W1; u.off_b1 = (unsigned)a->off_b1;
    u.off_W2 = (unsigned)(a->hidden ? a->off_W2 : a->nparam); u.off_b2 = (unsigned)(a->hidden ? a->off_b2 : a->nparam);
    u.nWc = (unsigned)z.nWc; u.nbc = (unsigned)z.F; u.nW1 = (unsigned)z.nW1; u.nb1 = (unsigned)z.nb1; u.nW2 = (unsigned)z.nW2; u.nb2 = (unsigned)z.nb2;
    u.slabs = slabs; u.slab_stride = (unsigned)slab_stride; u.nslab = nslab;
    u.head_partial = head_partial; u.nchunk = nchunk; u.pstride = pstride;
    u.nblock = (unsigned)a->nmodel; u.k = (unsigned)z.kt; u.h1 = (unsigned)(a->hidden ? a->hidden : 1); u.hidden = (unsigned)a->hidden;
    u.freeze_scan = a->freeze_scan; u.loss_kind = a->loss_kind; u.loss = a->loss; u.nrow = (unsigned)a->nregion;
    u.counter = (unsigned long long*)a->counter; u.counter_advance = draws;
    DBK_CHECK(z.nWc + z.F + z.nW1 + z.nb1 + z.nW2 + z.nb2 == a->nparam, "ValueError: the parameter blocks do not tile the flat vector (%zu of %zu elements)",
              z.nWc + z.F + z.nW1 + z.nb1 + z.nW2 + z.nb2, a->nparam);
    DBK_CHECK((head_partial != nullptr || a->nregion == 0) && slab_stride == z.nWc + z.F,
              "RuntimeError: the backward kernels left no partial sums");
    return 0;
}

}  // namespace

extern "C" int dbk_train_step(dbk_stream_t stream, const dbk_train_step_args* a)
{
    int rc = check_args(a);
    if (rc) return rc;
    const block_sizes z = sizes_of(a);
    const size_t F = z.F, k = z.k, nWc = z.nWc;

    // Nesterov with a look-ahead vector: the step's weights are read from L = P + mrate*mP, which the previous
    // step left there (L_ready) or which is formed now; otherwise the look-ahead is applied to P in place.
    const bool beside = a->nesterov && a->L != nullptr;
    float* const P = beside ? a->L : a->P;                         // where this step's weights are read
    float* const dP = a->dP;
    if (beside) {
        if (!a->L_ready) {
            rc = dbk_gradstep_lookahead(stream, DBK_F32, a->nparam, a->L, a->P, a->mP, a->mrate);
            if (rc) return rc;
        }
    } else if (a->nesterov) {
        rc = dbk_gradstep_nesterov1(stream, DBK_F32, a->nparam, P, a->mP, a->mrate);
        if (rc) return rc;
    }
    const uint8_t* X = a->X;
    if (a->input_rate > 0.0f) {
        rc = drop_inputs(stream, a);
        if (rc) return rc;
        X = a->Xdrop;
    }
    // with the look-ahead beside the parameters the backward kernels leave their partial sums for the step's last kernel
    dbk::deferred_sums later;
    struct scope { dbk::deferred_sums*& slot; ~scope() { slot = nullptr; } } guard{dbk::deferred()};
    if (beside) dbk::deferred() = &later;
    uint64_t* act = a->ptype == DBK_PT_MAX ? nullptr : a->act;      // only the average part of the backward pass reads the masks
    rc = dbk_scanpool_fprop(stream, P + a->off_Wc, P + a->off_bc, a->m, F, X, a->N, a->regions, a->nregion, a->ptype,
                            a->pooled, a->argmax, act);
    if (rc) return rc;
    const uint64_t draws = a->rate ? (a->nregion * k * a->nmodel + 3) / 4 : 0;
    rc = dbk_head_train(stream, a->nregion, (int)a->nmodel, (int)k, (int)a->hidden, a->loss_kind, a->reverse_complement,
                        a->pooled, (int)a->nfeat, a->feats, a->rate, nullptr, a->seed, 0, a->counter, draws,
                        P + a->off_W1, P + a->off_b1, a->hidden ? P + a->off_W2 : nullptr, a->hidden ? P + a->off_b2 : nullptr,
                        a->Y, a->Ymask, a->Z, a->dpooled,
                        dP + a->off_W1, dP + a->off_b1, a->hidden ? dP + a->off_W2 : nullptr, a->hidden ? dP + a->off_b2 : nullptr,
                        a->loss);
    if (rc) return rc;
    rc = dbk_scanpool_bprop(stream, P + a->off_Wc, P + a->off_bc, a->m, F, X, a->N, a->regions, a->nregion, a->ptype,
                            a->pooled, a->argmax, a->dpooled, dP + a->off_Wc, dP + a->off_bc, 1, act);
    if (rc) return rc;
    if (beside) {
        dbk::deferred() = nullptr;
        reduce_update_args u;
        rc = fill_update(u, a, z, later.slabs, later.slab_stride, later.nslab, later.head_partial, later.head_nchunk, later.head_pstride, draws);
        if (rc) return rc;
        hipLaunchKernelGGL(k_reduce_update, dim3(dbk::ew_grid(a->nparam + a->nmodel)), dim3(256), 0, dbk::as_stream(stream), u);
        DBK_LAUNCH_OK();
    }
    if (a->decay) {
        rc = dbk_l1_decay(stream, DBK_F32, P, a->decay, dP, a->nparam);
        if (rc) return rc;
    }
    if (a->freeze_scan) hipLaunchKernelGGL(k_zero_f32, dim3(dbk::ew_grid(nWc)), dim3(256), 0, dbk::as_stream(stream), dP + a->off_Wc, nWc);
    if (a->nesterov) rc = dbk_gradstep_nesterov2(stream, DBK_F32, a->nparam, P, dP, a->drate, a->mP, a->mrate);
    else rc = dbk_gradstep(stream, DBK_F32, a->nparam, P, dP, a->drate, a->mP, a->mrate);
    return rc;
}

// One step of each of several groups that train on the same batch: every phase of the step is ONE launch holding
// all the groups' grids, so groups too small to fill the GPU run side by side on one stream. A group's kernels,
// grids and summation orders are those of its own dbk_train_step, hence the same bits. Taken for up to 8 groups
// with a look-ahead vector each (Nesterov), filters of at most 24 taps and one shared region table; any other
// call steps the groups one after the other.
extern "C" int dbk_train_steps(dbk_stream_t stream, size_t ngroup, const dbk_train_step_args* const* args)
{
    DBK_CHECK(ngroup == 0 || args != nullptr, "ValueError: null argument list");
    for (size_t i = 0; i < ngroup; ++i) {
        int rc = check_args(args[i]);
        if (rc) return rc;
    }
    if (ngroup == 0) { dbk::clear_error(); return 0; }
    bool together = ngroup >= 2 && ngroup <= dbk::MULTI_MAX;
    const dbk_train_step_args* a0 = args[0];
    for (size_t i = 0; i < ngroup && together; ++i) {
        const dbk_train_step_args* a = args[i];
        together = a->nesterov && a->L && a->m == a0->m && a->N == a0->N && a->regions == a0->regions && a->nregion == a0->nregion &&
                   a->nregion > 0;
    }
    // dense (avg / max+avg) groups first: their workgroups run longest
    const dbk_train_step_args* ord[dbk::MULTI_MAX];
    dbk::scan_group sg[dbk::MULTI_MAX];
    if (together) {
        unsigned n = 0;
        for (int pass = 0; pass < 2; ++pass)
            for (size_t i = 0; i < ngroup; ++i)
                if ((args[i]->ptype == DBK_PT_MAX) == (pass == 1)) ord[n++] = args[i];
        for (unsigned i = 0; i < n; ++i) {
            const dbk_train_step_args* a = ord[i];
            const block_sizes z = sizes_of(a);
            sg[i].W = a->L + a->off_Wc; sg[i].bias = a->L + a->off_bc;
            sg[i].F = (unsigned)z.F; sg[i].ptype = a->ptype;
            sg[i].X = a->input_rate > 0.0f ? a->Xdrop : a->X;
            sg[i].pooled = a->pooled; sg[i].dpooled = a->dpooled; sg[i].argmax = a->argmax;
            sg[i].act = a->ptype == DBK_PT_MAX ? nullptr : reinterpret_cast<unsigned long long*>(a->act);
            sg[i].slabs = nullptr; sg[i].slab_stride = 0; sg[i].nslab = 0;
        }
        together = dbk::scan_multi_takes(a0->m, a0->N, a0->nregion, n, sg);
    }
    if (!together) {
        for (size_t i = 0; i < ngroup; ++i) {
            int rc = dbk_train_step(stream, args[i]);
            if (rc) return rc;
        }
        return 0;
    }
    const unsigned n = (unsigned)ngroup;
    hipStream_t st = dbk::as_stream(stream);
    int rc;
    // look-ahead vectors that the previous step did not leave
    {
        lookahead_multi_args la;
        la.n = 0; la.first[0] = 0;
        for (unsigned i = 0; i < n; ++i)
            if (!ord[i]->L_ready) {
                la.g[la.n] = { ord[i]->nparam, ord[i]->L, ord[i]->P, ord[i]->mP, ord[i]->mrate };
                la.first[la.n + 1] = la.first[la.n] + dbk::ew_grid(ord[i]->nparam);
                ++la.n;
            }
        if (la.n) hipLaunchKernelGGL(k_lookahead_multi, dim3(la.first[la.n]), dim3(256), 0, st, la);
    }
    for (unsigned i = 0; i < n; ++i)
        if (ord[i]->input_rate > 0.0f) {
            rc = drop_inputs(stream, ord[i]);
            if (rc) return rc;
        }
    rc = dbk::scan_fprop_multi(st, a0->m, a0->N, a0->regions, a0->nregion, n, sg);
    if (rc) return rc;
    dbk::head_group hg[dbk::MULTI_MAX];
    uint64_t draws[dbk::MULTI_MAX];
    for (unsigned i = 0; i < n; ++i) {
        const dbk_train_step_args* a = ord[i];
        const block_sizes z = sizes_of(a);
        const float* P = a->L;
        draws[i] = a->rate ? (a->nregion * z.k * a->nmodel + 3) / 4 : 0;
        hg[i].nblock = (int)a->nmodel; hg[i].k = (int)z.k; hg[i].kf = (int)a->nfeat; hg[i].feats = a->feats; hg[i].hidden = (int)a->hidden; hg[i].loss_kind = a->loss_kind;
        hg[i].revcomp = a->reverse_complement;
        hg[i].pooled = a->pooled; hg[i].rate = a->rate; hg[i].seed = a->seed; hg[i].counter = a->counter;
        hg[i].W1 = P + a->off_W1; hg[i].b1 = P + a->off_b1;
        hg[i].W2 = a->hidden ? P + a->off_W2 : nullptr; hg[i].b2 = a->hidden ? P + a->off_b2 : nullptr;
        hg[i].Y = a->Y; hg[i].Ymask = a->Ymask; hg[i].Z = a->Z; hg[i].dpooled = a->dpooled;
        hg[i].partial = nullptr; hg[i].nchunk = 0; hg[i].pstride = 0;
    }
    rc = dbk::head_train_multi(st, a0->nregion, n, hg);
    if (rc) return rc;
    rc = dbk::scan_bprop_multi(st, a0->m, a0->N, a0->regions, a0->nregion, n, sg);
    if (rc) return rc;
    reduce_update_multi_args um;
    um.n = n; um.first[0] = 0;
    for (unsigned i = 0; i < n; ++i) {
        const dbk_train_step_args* a = ord[i];
        rc = fill_update(um.g[i], a, sizes_of(a), sg[i].slabs, sg[i].slab_stride, sg[i].nslab, hg[i].partial, hg[i].nchunk, hg[i].pstride, draws[i]);
        if (rc) return rc;
        um.first[i + 1] = um.first[i] + dbk::ew_grid(a->nparam + a->nmodel);
    }
    hipLaunchKernelGGL(k_reduce_update_multi, dim3(um.first[n]), dim3(256), 0, st, um);
    DBK_LAUNCH_OK();
}

extern "C" int dbk_train_step_args_size(void) { return (int)sizeof(dbk_train_step_args); }
