// In-memory model runtime: the seam between MegCC's static memory plan and one HBM arena.
//
// A MegCC model is a list of tensors with byte offsets into ONE buffer, a list of weights and a
// list of `Opr` instructions, each naming a kernel and its tensors (runtime/schema/model.fbs:63-124,
// runtime/src/vm/instruction.h:61-76). The TinyNN runtime allocates that buffer once through
// Device.malloc and points every tensor at base + offset (runtime/src/init.c:437-487), runs the
// kernels' three-phase init on the weights (init.c:29-131) and then simply walks the instruction
// list (runtime/src/lite/network.c:171-227, vm/op.c:67-172). This file is that sequence with the
// gfx950 Device: weights are uploaded to HBM and repacked there by the kernels' init, the arena is
// one hipMalloc, input staging is a stream-ordered hipMemcpyAsync, and forward() is one
// asynchronous launch per Opr on the library stream.
//
// The MegCC compiler (and with it StaticMemoryPlanning) cannot be built without MLIR, so the plan
// is produced here from the same inputs it uses: per tensor the interval [defining opr, last
// using opr + 1) (compiler/lib/Dialect/Kernel/Transforms/StaticMemoryPlanning.cpp:88-96) and the
// byte size; tensors whose intervals overlap get disjoint offset ranges.
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <chrono>
#include <string>
#include <vector>

#include "common.h"
#include "memplan.h"
#include "tiny_reader.h"

using namespace mg;

namespace {

struct ModelTensor {
    Tensor t;
    std::string name;
    bool is_weight = false, is_input = false, is_output = false;
    int alias_of = -1;  // MemForward / reshape: shares the memory of another tensor
    size_t alias_offset = 0;  // MemForward: bytes from the start of that tensor
    int def = -1, last = -1;
    void* owned = nullptr;  // weights: device allocation owned by the model
};

struct ModelOpr {
    MegccKernelDesc desc;
    std::string symbol;
    std::vector<int> in, out;
    std::vector<Tensor*> in_ptrs, out_ptrs;
    Tensor processed;  // weight produced by the kernel's init, replaces one input
    bool has_processed = false;
    void* processed_mem = nullptr;
    Workspace ws;
    int first_index = -1;  // index in Model::oprs of the (first) operator this schedule entry stands for
};

struct Model {
    Device dev;
    RuntimeOpt opt;
    std::vector<ModelTensor*> tensors;
    std::vector<ModelOpr*> oprs;
    // what forward() launches: the operators in order, with recognised operator chains replaced by
    // one kernel (`fused` owns the replacements); run_opr, nr_opr and the memory plan keep the
    // operator list as it was given
    std::vector<ModelOpr*> schedule, fused;
    void* arena = nullptr;
    size_t arena_bytes = 0;
    // one scratch buffer shared by all operators (they run one after the other on one stream),
    // sized for the largest request of any operator's _workspace function
    void* workspace = nullptr;
    size_t workspace_bytes = 0;
    bool finalized = false;
    // offsets and arena size come from a model file (the compiler's static memory plan) instead
    // of plan_memory(); model inputs then live outside the arena, as in the TinyNN runtime
    bool preplanned = false;
    // The operator sequence of a finalized model never changes (static shapes, static memory plan),
    // so it can be captured once into a HIP graph and replayed: one launch per forward instead of one
    // per operator. 0: not decided yet, 1: graph in use, -1: eager (measured faster, capture failed,
    // a schedule of fewer than 5 kernels, or switched off by MEGCC_NO_GRAPH).
    // Whether replaying wins is MEASURED: a graph launch costs about 13 us before its first kernel
    // starts, eager launches cost the host 3-4 us per kernel, so small batches (host-bound) gain from
    // the graph and large ones lose its fixed cost. Forward 1 runs eagerly (it warms per-kernel
    // attributes), 2 and 3 eagerly between two events, 4 captures and launches, 5 and 6 replay between
    // the events; from forward 7 on the faster way is used.
    int graph_state = 0;
    int forwards = 0;
    float eager_ms = 1e30f, graph_ms = 1e30f;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t graph_exec = nullptr;
    // Consecutive forwards overlap: the last operators of a network are small (a few megabytes, a
    // launch floor each) and the first operators of the next forward do not depend on them, so with
    // plain launches the schedule from `tail_begin` on runs on a second stream, ordered behind the head
    // by an event, while the library stream is free for the next forward's head. `tail_opr_begin` is
    // the same boundary in `oprs` (chosen before the memory plan, which then gives every tensor the
    // tail touches bytes of its own); `waits_tail[i]`: head entry i writes bytes the previous
    // forward's tail may still be using and waits for it first (under the runtime's own plan that is
    // only the entry that produces the tail's input). The tail has its own workspace.
    int tail_opr_begin = -1, tail_begin = -1;
    hipStream_t tail_stream = nullptr;
    hipEvent_t ev_head = nullptr, ev_tail = nullptr;
    bool tail_pending = false, tail_reads_input = false;
    std::vector<char> waits_tail;
    std::vector<const Tensor*> tail_writes;  // tensors the tail's operators write
    void* tail_workspace = nullptr;
};

size_t tensor_bytes(const Tensor& t) {
    return nr_elem(t.layout) * dtype_size(&t);
}

size_t align_up(size_t v, size_t a) {
    return (v + a - 1) / a * a;
}

int root_of(const Model* m, int id) {
    while (m->tensors[id]->alias_of >= 0)
        id = m->tensors[id]->alias_of;
    return id;
}

// Offsets for the arena from the tensors' lifetimes: time step = operator index, a tensor is
// alive from the operator that writes it to one past the last operator that reads it
// (compiler/lib/Dialect/Kernel/Transforms/StaticMemoryPlanning.cpp:88-96). Model inputs are not
// planned: the compiler plans allocations only and the function arguments are the caller's memory
// (runtime/src/init.c:456-460); here each input is a device buffer of its own, which keeps what
// set_input put there across any number of forwards. Outputs stay valid after forward().
// Where the tail of a forward may begin (see Model::tail_begin): the longest suffix of the operator
// list estimated to take at most 55 % of the forward - the two streams should end up with about the
// same amount of work, which is where back-to-back forwards gain most (MobileNetV1: the split falls
// behind the 28 x 28 layers at every batch from 16 to 128); setup_tail() shortens it to the measured
// balance - with a head of at least four operators, a tail of at least two, and at most `own_cap`
// bytes of tensors in the tail (they get bytes of their own in the memory plan). The estimate is a launch
// floor plus the operator's tensors at half the memory bandwidth.
static void choose_tail(Model* m, size_t own_cap) {
    m->tail_opr_begin = -1;
    if (options().no_pipeline)
        return;
    const int n = (int)m->oprs.size();
    std::vector<double> us((size_t)n);
    double total = 0;
    for (int i = 0; i < n; ++i) {
        size_t bytes = 0;
        for (int id : m->oprs[i]->in)
            bytes += tensor_bytes(m->tensors[id]->t);
        for (int id : m->oprs[i]->out)
            bytes += tensor_bytes(m->tensors[id]->t);
        us[(size_t)i] = 3.8 + (double)bytes / 4.0e6;
        total += us[(size_t)i];
    }
    std::vector<char> seen(m->tensors.size(), 0);
    size_t own = 0;
    double tail = 0;
    int k = n;
    while (k > 4 && tail + us[(size_t)k - 1] <= 0.55 * total) {
        const ModelOpr* o = m->oprs[k - 1];
        size_t more = 0;
        for (const std::vector<int>* ids : {&o->in, &o->out})
            for (int id : *ids) {
                const int r = root_of(m, id);
                if (!seen[r] && !m->tensors[r]->is_weight && !m->tensors[r]->is_input) {
                    seen[r] = 1;
                    more += tensor_bytes(m->tensors[r]->t);
                }
            }
        if (own + more > own_cap)
            break;
        own += more;
        tail += us[(size_t)k - 1];
        --k;
    }
    if (n - k >= 2)
        m->tail_opr_begin = k;
}

bool plan_memory(Model* m) {
    if (m->preplanned)
        return true;
    // A pointwise convolution followed by the channel-wise 3x3 convolution of its result may run
    // as one kernel (build_schedule), which reads the pointwise layer's source while it writes the
    // channel-wise layer's result: that source stays alive one operator longer, as it would in a
    // plan made for the one operator.
    std::vector<int> keep_until(m->tensors.size(), -1);
    for (size_t i = 0; !options().no_fuse_pwdw && i + 1 < m->oprs.size(); ++i) {
        const ModelOpr *o0 = m->oprs[i], *o1 = m->oprs[i + 1];
        if (o0->desc.kind != MEGCC_KERN_CONV || o1->desc.kind != MEGCC_KERN_CONV || o0->in.empty() ||
            o1->in.empty() || o0->out.size() != 1 || o1->in[0] != o0->out[0])
            continue;
        const MegccConvAttr &a = o0->desc.attr.conv, &b = o1->desc.attr.conv;
        if (a.format == MEGCC_FMT_NCHW44 && a.sparse == MEGCC_SPARSE_DENSE && a.kernel_h == 1 && a.kernel_w == 1 &&
            a.stride_h == 1 && a.stride_w == 1 && a.pad_h == 0 && a.pad_w == 0 && b.format == MEGCC_FMT_NCHW44 &&
            b.sparse == MEGCC_SPARSE_GROUP && b.kernel_h == 3 && b.kernel_w == 3 && b.pad_h == 1 && b.pad_w == 1) {
            // ... where the one kernel can win at all: shapes it takes, and no more images than give
            // every CU a workgroup or two (beyond that the two kernels are faster, and a longer
            // lifetime only costs arena and cache reuse)
            const Layout& sl = m->tensors[o0->in[0]]->t.layout;
            const Layout& ml = m->tensors[o0->out[0]]->t.layout;
            if (sl.nr_dim != 5 || ml.nr_dim != 5)
                continue;
            const long n = sl.dims[0], ic = 4L * sl.dims[1], w = sl.dims[3], oc = 4L * ml.dims[1];
            if ((ic == 128 || ic == 256 || ic == 512) && oc % 64 == 0 && w >= 4 && w <= 31 && n * (oc / 64) <= 512)
                keep_until[root_of(m, o0->in[0])] = (int)i + 1;
        }
    }
    // What the tail of a forward touches shares no byte with anything else: the head of the next
    // forward runs while the tail is still at work.
    std::vector<char> pinned(m->tensors.size(), 0);
    for (size_t i = m->tail_opr_begin < 0 ? m->oprs.size() : (size_t)m->tail_opr_begin; i < m->oprs.size(); ++i) {
        for (int id : m->oprs[i]->in)
            pinned[root_of(m, id)] = 1;
        for (int id : m->oprs[i]->out)
            pinned[root_of(m, id)] = 1;
    }
    std::vector<MemInterval> intervals;
    std::vector<int> ids;
    for (size_t i = 0; i < m->tensors.size(); ++i) {
        ModelTensor* t = m->tensors[i];
        if (t->is_weight || t->is_input || t->alias_of >= 0 || t->def < 0)
            continue;
        MemInterval iv;
        iv.begin = pinned[i] ? 0 : (size_t)t->def;
        iv.end = t->is_output || pinned[i] ? m->oprs.size() + 1 : (size_t)std::max(t->last, keep_until[i]) + 1;
        iv.size = tensor_bytes(t->t);
        intervals.push_back(iv);
        ids.push_back((int)i);
    }
    std::vector<size_t> offsets;
    size_t total = 0;
    if (!plan_memory_pushdown(intervals, m->dev.alignment, &offsets, &total, nullptr))
        return false;
    for (size_t k = 0; k < ids.size(); ++k)
        m->tensors[ids[k]]->t.offset = offsets[k];
    m->arena_bytes = total;
    return true;
}

// ---- forward schedule ----------------------------------------------------------------------------
// The importer's decomposition of a soft-max (Reduce MAX over the last axis -> SUB -> EXP -> Reduce
// SUM -> TRUE_DIV, compiler/lib/Target/MGB/importer.cpp:987-1016), optionally behind the typecvt
// qsi8 -> f32 that dequantises the logits, is five or six kernel boundaries of 3-5 us each for half
// a megabyte of data. When the intermediate tensors have no other reader and are no outputs, the
// chain runs as ONE kernel (softmax.hip). The intermediates keep their place in the memory plan.
static bool dense_f32(const Tensor& t) {
    return t.dtype.type_enum == TinyNN_FLOAT && is_contiguous(t.layout);
}
// [ptr, ptr + bytes) of a dense tensor against another's: the kernels that replace an operator chain
// read their inputs while other workgroups already write the chain's output, which is only safe
// when the two ranges share no byte. A memory plan made for the unfused operators (the compiler's,
// or plan_memory() above) may well put the chain's output into bytes an input of the chain's first
// operator has just freed.
static bool shares_bytes(const Tensor& a, const Tensor& b) {
    const char *a0 = (const char*)a.ptr, *b0 = (const char*)b.ptr;
    const size_t an = tensor_bytes(a), bn = tensor_bytes(b);
    if (!a0 || !b0 || !an || !bn)
        return false;
    return a0 < b0 + bn && b0 < a0 + an;
}
// Milliseconds `iters` back-to-back rounds of the operators in `ops` take on the library stream
// (after one untimed round), or a negative value when a launch fails or an operand has no memory.
static float time_oprs(Model* m, const std::vector<ModelOpr*>& ops, int iters) {
    for (const ModelOpr* o : ops) {
        for (const Tensor* t : o->in_ptrs)
            if (!t->ptr)
                return -1.f;
        for (const Tensor* t : o->out_ptrs)
            if (!t->ptr)
                return -1.f;
    }
    auto round = [&]() {
        for (ModelOpr* o : ops)
            if (megcc_gfx950_call(
                        &o->desc, o->in_ptrs.data(), (int)o->in_ptrs.size(), o->out_ptrs.data(),
                        (int)o->out_ptrs.size(), &o->ws, &m->opt) != TinyNN_SUCCESS)
                return false;
        return true;
    };
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        if (e0)
            (void)hipEventDestroy(e0);
        return -1.f;
    }
    float ms = -1.f;
    bool ok = round();
    ok = ok && hipEventRecord(e0, stream()) == hipSuccess;
    for (int i = 0; ok && i < iters; ++i)
        ok = round();
    ok = ok && hipEventRecord(e1, stream()) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
         hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return ok ? ms : -1.f;
}

static void build_schedule(Model* m, bool allow_pw_dw = true) {
    m->schedule.clear();
    const int n = (int)m->oprs.size();
    for (int i = 0; i < n; ++i)
        m->oprs[i]->first_index = i;
    std::vector<int> readers(m->tensors.size(), 0);
    for (auto* o : m->oprs)
        for (int id : o->in)
            ++readers[root_of(m, id)];
    // a tensor only this chain touches: its own memory, `nr` readers, neither input, output nor weight
    auto temp = [&](int id, int nr) {
        const ModelTensor* t = m->tensors[id];
        return t->alias_of < 0 && !t->is_input && !t->is_output && !t->is_weight && readers[id] == nr;
    };
    auto is_ew = [](const ModelOpr* o, MegccElemwiseMode mode, size_t nin) {
        return o->desc.kind == MEGCC_KERN_ELEMWISE && o->desc.attr.elemwise == mode &&
               o->in.size() == nin && o->out.size() == 1;
    };
    auto is_red = [&](const ModelOpr* o, MegccReduceMode mode) {
        if (o->desc.kind != MEGCC_KERN_REDUCE || o->desc.attr.reduce.mode != mode ||
            o->in.size() != 1 || o->out.size() != 1)
            return false;
        const Tensor& s = m->tensors[o->in[0]]->t;
        return o->desc.attr.reduce.axis == s.layout.nr_dim - 1;
    };
    for (int i = 0; i < n; ++i) {
        ModelOpr* o0 = m->oprs[i];
        // A channel-wise 3x3 convolution, the 2x2 stride-2 maximum pooling of its result and the
        // quantised addition of the pooled tensor with another one: all three are bound by memory
        // traffic, and two thirds of it is the two tensors in between going out and coming back.
        // When nothing else reads those, the chain runs as ONE kernel (megcc_gfx950_dw_pool_add).
        if (!options().no_fuse_chain && i + 2 < n && o0->desc.kind == MEGCC_KERN_CONV && !o0->has_processed &&
            o0->out.size() == 1) {
            ModelOpr *o1 = m->oprs[i + 1], *o2 = m->oprs[i + 2];
            if (o1->desc.kind == MEGCC_KERN_POOLING && o1->in.size() == 1 && o1->out.size() == 1 &&
                o1->in[0] == o0->out[0] && o2->desc.kind == MEGCC_KERN_ELEMWISE_MULTITYPE && o2->in.size() == 2 &&
                o2->out.size() == 1 && (o2->in[0] == o1->out[0]) != (o2->in[1] == o1->out[0]) &&
                temp(o0->out[0], 1) && temp(o1->out[0], 1) &&
                m->tensors[o0->out[0]]->t.dtype.param.scale == m->tensors[o1->out[0]]->t.dtype.param.scale) {
                const int other = o2->in[0] == o1->out[0] ? o2->in[1] : o2->in[0];
                ModelOpr* f = new ModelOpr();
                f->first_index = i;
                memset(&f->desc, 0, sizeof(f->desc));
                f->desc.kind = MEGCC_KERN_DW_POOL_ADD;
                f->desc.attr.dw_pool_add.conv = o0->desc.attr.conv;
                f->desc.attr.dw_pool_add.pool = o1->desc.attr.pool;
                f->desc.attr.dw_pool_add.mode = o2->desc.attr.multitype;
                f->desc.attr.dw_pool_add.mid_scale = m->tensors[o0->out[0]]->t.dtype.param.scale;
                f->symbol = "depthwise 3x3 + max-pool 2x2 + add (fused)";
                memset(&f->ws, 0, sizeof(f->ws));
                f->in = o0->in;
                f->in_ptrs = o0->in_ptrs;
                f->in.push_back(other);
                f->in_ptrs.push_back(&m->tensors[other]->t);
                f->out = o2->out;
                f->out_ptrs = o2->out_ptrs;
                // the kernel reads src (with halos) and `other` while it writes the output
                bool apart = true;
                for (const Tensor* t : f->in_ptrs)
                    apart = apart && !shares_bytes(*t, *f->out_ptrs[0]);
                if (apart && megcc_gfx950_dw_pool_add_supported(
                            &f->desc.attr.dw_pool_add, f->in_ptrs.data(), (int)f->in_ptrs.size(), f->out_ptrs.data(),
                            (int)f->out_ptrs.size())) {
                    m->fused.push_back(f);
                    m->schedule.push_back(f);
                    i += 2;
                    continue;
                }
                delete f;
            }
        }
        // A pointwise convolution and the channel-wise 3x3 convolution of its result, on images small
        // enough for a workgroup to hold one: one kernel (megcc_gfx950_pw_dw) when nothing else reads
        // the tensor in between.
        if (allow_pw_dw && !options().no_fuse_pwdw && i + 1 < n && o0->desc.kind == MEGCC_KERN_CONV && o0->has_processed &&
            o0->out.size() == 1 && o0->in.size() == (o0->desc.attr.conv.with_bias ? 3u : 2u)) {
            ModelOpr* o1 = m->oprs[i + 1];
            if (o1->desc.kind == MEGCC_KERN_CONV && !o1->has_processed && o1->out.size() == 1 &&
                o1->in.size() == (o1->desc.attr.conv.with_bias ? 3u : 2u) && o1->in[0] == o0->out[0] &&
                o1->desc.attr.conv.sparse == MEGCC_SPARSE_GROUP && temp(o0->out[0], 1)) {
                ModelOpr* f = new ModelOpr();
                f->first_index = i;
                memset(&f->desc, 0, sizeof(f->desc));
                f->desc.kind = MEGCC_KERN_PW_DW;
                f->desc.attr.pw_dw.pw = o0->desc.attr.conv;
                f->desc.attr.pw_dw.dw = o1->desc.attr.conv;
                f->desc.attr.pw_dw.mid_scale = m->tensors[o0->out[0]]->t.dtype.param.scale;
                f->symbol = "pointwise 1x1 + depthwise 3x3 (fused)";
                memset(&f->ws, 0, sizeof(f->ws));
                f->in = o0->in;
                f->in_ptrs = o0->in_ptrs;
                for (size_t k = 1; k < o1->in.size(); ++k) {
                    f->in.push_back(o1->in[k]);
                    f->in_ptrs.push_back(o1->in_ptrs[k]);
                }
                f->out = o1->out;
                f->out_ptrs = o1->out_ptrs;
                // a workgroup reads its whole image before it stores, but other images' workgroups
                // run at the same time: source and result must share no byte
                bool take = !shares_bytes(*f->in_ptrs[0], *f->out_ptrs[0]) &&
                            megcc_gfx950_pw_dw_supported(
                                    &f->desc.attr.pw_dw, f->in_ptrs.data(), (int)f->in_ptrs.size(),
                                    f->out_ptrs.data(), (int)f->out_ptrs.size());
                // The one kernel saves a launch and the tensor's round trip, but its three phases run
                // one after the other on a CU, so which form is faster depends on how many images
                // there are per CU: both forms are run a few times on the tensors as they are (their
                // contents do not matter before the first forward) and the faster one is kept. The
                // switch "fusepwdw" takes the one kernel without measuring.
                if (take && !options().fuse_pwdw) {
                    const float one = time_oprs(m, {f}, 20), two = time_oprs(m, {o0, o1}, 20);
                    take = one > 0.f && two > 0.f && one < 0.97f * two;
                }
                if (take) {
                    m->fused.push_back(f);
                    m->schedule.push_back(f);
                    i += 1;
                    continue;
                }
                delete f;
            }
        }
        bool fuse = !options().no_fuse_softmax && i + 4 < n && is_red(o0, MEGCC_REDUCE_MAX) &&
                    is_ew(m->oprs[i + 1], MEGCC_EW_SUB, 2) && is_ew(m->oprs[i + 2], MEGCC_EW_EXP, 1) &&
                    is_red(m->oprs[i + 3], MEGCC_REDUCE_SUM) && is_ew(m->oprs[i + 4], MEGCC_EW_TRUE_DIV, 2);
        if (fuse) {
            ModelOpr *o1 = m->oprs[i + 1], *o2 = m->oprs[i + 2], *o3 = m->oprs[i + 3], *o4 = m->oprs[i + 4];
            const int x = o0->in[0], mx = o0->out[0], sub = o1->out[0], ex = o2->out[0], sum = o3->out[0],
                      y = o4->out[0];
            const Tensor& tx = m->tensors[x]->t;
            const Tensor& ty = m->tensors[y]->t;
            const size_t cols = tx.layout.nr_dim ? tx.layout.dims[tx.layout.nr_dim - 1] : 0;
            fuse = o1->in[0] == x && o1->in[1] == mx && o2->in[0] == sub && o3->in[0] == ex &&
                   o4->in[0] == ex && o4->in[1] == sum && m->tensors[x]->alias_of < 0 &&
                   m->tensors[y]->alias_of < 0 && temp(mx, 1) && temp(sub, 1) && temp(ex, 2) &&
                   temp(sum, 1) && dense_f32(tx) && dense_f32(ty) && dense_f32(m->tensors[mx]->t) &&
                   dense_f32(m->tensors[sum]->t) && dense_f32(m->tensors[sub]->t) &&
                   dense_f32(m->tensors[ex]->t) && cols >= 1 &&
                   cols <= (size_t)megcc_gfx950_softmax_max_columns() &&
                   nr_elem(ty.layout) == nr_elem(tx.layout) &&
                   nr_elem(m->tensors[sub]->t.layout) == nr_elem(tx.layout) &&
                   nr_elem(m->tensors[ex]->t.layout) == nr_elem(tx.layout) &&
                   nr_elem(m->tensors[mx]->t.layout) * cols == nr_elem(tx.layout) &&
                   nr_elem(m->tensors[sum]->t.layout) * cols == nr_elem(tx.layout);
            if (fuse) {
                int src = x;
                // the dequantisation in front of it, when the soft-max is all that reads its result
                if (!m->schedule.empty() && i > 0 && m->schedule.back() == m->oprs[i - 1]) {
                    const ModelOpr* cv = m->oprs[i - 1];
                    if (cv->desc.kind == MEGCC_KERN_TYPECVT && cv->in.size() == 1 && cv->out.size() == 1 &&
                        cv->out[0] == x && temp(x, 2) &&
                        m->tensors[cv->in[0]]->t.dtype.type_enum == TinyNN_QINT8 &&
                        is_contiguous(m->tensors[cv->in[0]]->t.layout) &&
                        nr_elem(m->tensors[cv->in[0]]->t.layout) == nr_elem(tx.layout) &&
                        // (only when the qsi8 logits and the result share no byte: a row of the
                        //  result covers four rows' worth of logit bytes)
                        !shares_bytes(m->tensors[cv->in[0]]->t, ty)) {
                        src = cv->in[0];
                        m->schedule.pop_back();
                    }
                }
                // A row is read whole before it is written, by one workgroup, so a result that
                // starts exactly where its f32 source starts is fine; any other overlap would let
                // one row's stores land in another row's unread source.
                const Tensor& ts = m->tensors[src]->t;
                if (shares_bytes(ts, ty) && !(src == x && ts.ptr == ty.ptr)) {
                    m->schedule.push_back(o0);
                    continue;
                }
                ModelOpr* f = new ModelOpr();
                f->first_index = i;
                memset(&f->desc, 0, sizeof(f->desc));
                f->desc.kind = MEGCC_KERN_SOFTMAX;
                f->symbol = "softmax (fused)";
                if (src != x)
                    f->first_index = i - 1;  // (the dequantisation in front joined)
                memset(&f->ws, 0, sizeof(f->ws));
                f->in.push_back(src);
                f->out.push_back(y);
                f->in_ptrs.push_back(&m->tensors[src]->t);
                f->out_ptrs.push_back(&m->tensors[y]->t);
                m->fused.push_back(f);
                m->schedule.push_back(f);
                i += 4;
                continue;
            }
        }
        m->schedule.push_back(o0);
    }
}

// The tail stream, its events and workspace, and which head entries must wait for the previous
// forward's tail (see Model::tail_begin). Leaves tail_begin at -1 when there is nothing to overlap.
// `forced`: the boundary to use (a schedule index; finalize tries the neighbours of the balanced one).
static void setup_tail(Model* m, int forced = -1) {
    m->tail_begin = -1;
    if (m->tail_opr_begin < 0)
        return;
    const int n = (int)m->schedule.size();
    int tb = -1;
    for (int s = 0; s < n; ++s)
        if (m->schedule[s]->first_index >= m->tail_opr_begin) {
            tb = s;
            break;
        }
    if (tb < 1 || tb >= n)
        return;
    if (forced >= 0) {
        if (forced < 1 || forced > n - 2)
            return;
        tb = forced;
    } else
    // The boundary the memory plan was made for came from an estimate; with the kernels at hand each
    // entry is timed (a few launches on the tensors as they are; the estimate stands in for an entry
    // that cannot be run) and the tail is shortened until it takes no
    // longer than the head: one fused pair too many on the tail costs MobileNetV1 batch 64 3 %.
    {
        std::vector<double> us((size_t)n);
        double total = 0;
        for (int s = 0; s < n; ++s) {
            ModelOpr* o = m->schedule[(size_t)s];
            const float ms = time_oprs(m, {o}, 8);
            if (ms > 0.f) {
                us[(size_t)s] = ms * 1e3 / 8;
            } else {
                size_t bytes = 0;
                for (const Tensor* t : o->in_ptrs)
                    bytes += tensor_bytes(*t);
                for (const Tensor* t : o->out_ptrs)
                    bytes += tensor_bytes(*t);
                us[(size_t)s] = 3.8 + (double)bytes / 4.0e6;
            }
            total += us[(size_t)s];
        }
        // A network whose kernels average under 6 us is bound by launches, not by the device: two
        // streams then gain or lose a quarter from run to run (MobileNetV1 batch 1: 7.2 k ... 9.9 k
        // img/s) where one stream or a graph replay is steady. One stream.
        if (total < 6.0 * n)
            return;
        double tail = 0;
        for (int s = tb; s < n; ++s)
            tail += us[(size_t)s];
        while (tb < n - 2 && tail > total - tail) {
            tail -= us[(size_t)tb];
            ++tb;
        }
    }
    // every tensor the tail reads or writes (weights are never written by anyone)
    std::vector<const Tensor*> touched;
    size_t ws_bytes = 0;
    for (int s = tb; s < n; ++s) {
        const ModelOpr* o = m->schedule[s];
        for (const Tensor* t : o->in_ptrs)
            if (!t->is_weight) {
                touched.push_back(t);
                m->tail_reads_input = m->tail_reads_input || t->is_input;
            }
        for (const Tensor* t : o->out_ptrs) {
            touched.push_back(t);
            m->tail_writes.push_back(t);
        }
        ws_bytes = std::max(ws_bytes, (size_t)o->ws.size);
    }
    if (hipStreamCreateWithFlags(&m->tail_stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&m->ev_head, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&m->ev_tail, hipEventDisableTiming) != hipSuccess)
        return;
    if (ws_bytes) {
        m->tail_workspace = m->dev.malloc(ws_bytes);
        if (!m->tail_workspace)
            return;
        for (int s = tb; s < n; ++s)
            if (m->schedule[s]->ws.size)
                m->schedule[s]->ws.ptr = m->tail_workspace;
    }
    m->waits_tail.assign((size_t)tb, 0);
    for (int s = 0; s < tb; ++s)
        for (const Tensor* w : m->schedule[s]->out_ptrs)
            for (const Tensor* t : touched)
                if (shares_bytes(*w, *t))
                    m->waits_tail[(size_t)s] = 1;
    register_aux_stream(m->tail_stream);
    m->tail_begin = tb;
}

// Makes the library stream wait for the tail of the last forward (nothing to do when there is none).
static void join_tail(Model* m) {
    if (m->tail_pending) {
        (void)hipStreamWaitEvent(main_stream(), m->ev_tail, 0);
        m->tail_pending = false;
    }
}

// Undoes setup_tail (the schedule is about to be rebuilt).
static void reset_tail(Model* m) {
    if (m->tail_stream) {
        (void)hipStreamSynchronize(m->tail_stream);
        unregister_aux_stream(m->tail_stream);
        (void)hipStreamDestroy(m->tail_stream);
        m->tail_stream = nullptr;
    }
    if (m->ev_head)
        (void)hipEventDestroy(m->ev_head);
    if (m->ev_tail)
        (void)hipEventDestroy(m->ev_tail);
    m->ev_head = m->ev_tail = nullptr;
    if (m->tail_workspace)
        m->dev.free(m->tail_workspace);
    m->tail_workspace = nullptr;
    for (auto* o : m->oprs)
        o->ws.ptr = o->ws.size ? m->workspace : nullptr;
    m->waits_tail.clear();
    m->tail_writes.clear();
    m->tail_reads_input = m->tail_pending = false;
    m->tail_begin = -1;
}

// LITE_forward: one asynchronous kernel launch per Opr, in order, on the library stream; stops at
// the first failing kernel like network.c:191-194. Results are visible after megcc_gfx950_wait().
// `overlap`: the entries from tail_begin on go to the tail stream (plain launches of a model whose way
// of launching is decided; never under capture or between timing events).
// `done`: an event recorded behind the forward's last operator, on whichever stream that is.
static TinyNNStatus forward_eager(Model* m, bool overlap = false, hipEvent_t done = nullptr) {
    const int tb = overlap ? m->tail_begin : -1;
    if (tb < 0)
        join_tail(m);
    TinyNNStatus st = TinyNN_SUCCESS;
    for (int idx = 0; idx < (int)m->schedule.size() && st == TinyNN_SUCCESS; ++idx) {
        ModelOpr* o = m->schedule[(size_t)idx];
        if (idx == tb) {
            (void)hipEventRecord(m->ev_head, main_stream());
            (void)hipStreamWaitEvent(m->tail_stream, m->ev_head, 0);
            set_stream_override(m->tail_stream, true);
        } else if (idx < tb && m->tail_pending && m->waits_tail[(size_t)idx]) {
            join_tail(m);
        }
        st = megcc_gfx950_call(
                &o->desc, o->in_ptrs.data(), (int)o->in_ptrs.size(), o->out_ptrs.data(),
                (int)o->out_ptrs.size(), &o->ws, &m->opt);
    }
    if (tb >= 0) {
        set_stream_override(nullptr, false);
        (void)hipEventRecord(m->ev_tail, m->tail_stream);
        m->tail_pending = true;
    }
    if (done)
        (void)hipEventRecord(done, tb >= 0 ? m->tail_stream : main_stream());
    return st;
}

// Milliseconds per forward of eight plain-launch forwards enqueued back to back, the way a finalized
// model runs them (two streams where the schedule has a tail) - the shorter of two such runs;
// negative when something fails.
static float time_forwards(Model* m) {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        if (e0)
            (void)hipEventDestroy(e0);
        return -1.f;
    }
    float best = -1.f;
    bool ok = forward_eager(m) == TinyNN_SUCCESS;
    for (int rep = 0; ok && rep < 2; ++rep) {
        float ms = -1.f;
        join_tail(m);
        ok = hipEventRecord(e0, main_stream()) == hipSuccess;
        for (int i = 0; ok && i < 8; ++i)
            ok = forward_eager(m, true) == TinyNN_SUCCESS;
        join_tail(m);
        ok = ok && hipEventRecord(e1, main_stream()) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
             hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
        if (ok && (best < 0.f || ms / 8 < best))
            best = ms / 8;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return ok ? best : -1.f;
}

}  // namespace

extern "C" {

void* megcc_gfx950_model_create(void) {
    Model* m = new Model();
    if (megcc_gfx950_init_device(&m->dev) != TinyNN_SUCCESS) {
        delete m;
        return nullptr;
    }
    m->opt.device = &m->dev;
    return m;
}

void megcc_gfx950_model_destroy(void* model) {
    Model* m = (Model*)model;
    if (!m)
        return;
    (void)hipStreamSynchronize(stream());
    if (m->tail_stream) {
        (void)hipStreamSynchronize(m->tail_stream);
        unregister_aux_stream(m->tail_stream);
        (void)hipStreamDestroy(m->tail_stream);
    }
    if (m->ev_head)
        (void)hipEventDestroy(m->ev_head);
    if (m->ev_tail)
        (void)hipEventDestroy(m->ev_tail);
    if (m->tail_workspace)
        m->dev.free(m->tail_workspace);
    for (auto* o : m->oprs) {
        if (o->processed_mem)
            m->dev.free(o->processed_mem);
        delete o;
    }
    for (auto* t : m->tensors) {
        if (t->owned)
            m->dev.free(t->owned);
        delete t;
    }
    for (auto* o : m->fused)
        delete o;
    if (m->arena)
        m->dev.free(m->arena);
    if (m->workspace)
        m->dev.free(m->workspace);
    if (m->ev0)
        (void)hipEventDestroy(m->ev0);
    if (m->ev1)
        (void)hipEventDestroy(m->ev1);
    if (m->graph_exec)
        (void)hipGraphExecDestroy(m->graph_exec);
    if (m->graph)
        (void)hipGraphDestroy(m->graph);
    delete m;
}

static int add_tensor(
        Model* m, const char* name, int nr_dim, const uint32_t* dims, TinyNNDType dtype,
        float scale) {
    if (!m || m->finalized || nr_dim < 1 || nr_dim > MAX_DIM || !dims)
        return -1;
    ModelTensor* t = new ModelTensor();
    memset(&t->t, 0, sizeof(Tensor));
    t->name = name ? name : "";
    t->t.dtype.type_enum = dtype;
    t->t.dtype.param.scale = scale;
    t->t.layout.nr_dim = nr_dim;
    int stride = 1;
    for (int i = nr_dim - 1; i >= 0; --i) {
        t->t.layout.dims[i] = dims[i];
        t->t.layout.stride[i] = stride;
        stride *= dims[i];
    }
    t->t.size = tensor_bytes(t->t);
    m->tensors.push_back(t);
    t->t.name = (char*)m->tensors.back()->name.c_str();
    return (int)m->tensors.size() - 1;
}

int megcc_gfx950_model_add_tensor(
        void* model, const char* name, int nr_dim, const uint32_t* dims, TinyNNDType dtype,
        float scale) {
    return add_tensor((Model*)model, name, nr_dim, dims, dtype, scale);
}

int megcc_gfx950_model_add_weight(
        void* model, const char* name, int nr_dim, const uint32_t* dims, TinyNNDType dtype,
        float scale, const void* host_data) {
    Model* m = (Model*)model;
    int id = add_tensor(m, name, nr_dim, dims, dtype, scale);
    if (id < 0 || !host_data)
        return -1;
    ModelTensor* t = m->tensors[id];
    t->is_weight = true;
    t->t.is_weight = 1;
    t->owned = m->dev.malloc(t->t.size);
    if (!t->owned)
        return -1;
    t->t.ptr = t->owned;
    if (megcc_gfx950_memcpy_h2d(t->owned, host_data, t->t.size) != TinyNN_SUCCESS)
        return -1;
    return id;
}

int megcc_gfx950_model_add_alias(
        void* model, const char* name, int of, int nr_dim, const uint32_t* dims) {
    Model* m = (Model*)model;
    if (!m || of < 0 || of >= (int)m->tensors.size())
        return -1;
    const Tensor& src = m->tensors[of]->t;
    int id = add_tensor(m, name, nr_dim, dims, src.dtype.type_enum, src.dtype.param.scale);
    if (id < 0)
        return -1;
    if (tensor_bytes(m->tensors[id]->t) != tensor_bytes(src)) {
        fail(TinyNN_ERROR_INVALID_LAYOUT, "model_add_alias: byte sizes differ");
        return -1;
    }
    m->tensors[id]->alias_of = of;
    return id;
}

// A strided window into tensor `of` (what the compiler's SUBTENSOR / DIMSHUFFLE MemForward
// leaves in a model, runtime/schema/model.fbs:125-140): dims and strides (elements) of the view,
// its first element `offset_bytes` after the start of `of`. Every element must lie inside `of`.
int megcc_gfx950_model_add_view(
        void* model, const char* name, int of, int nr_dim, const uint32_t* dims,
        const int* strides, size_t offset_bytes) {
    Model* m = (Model*)model;
    if (!m || !strides || of < 0 || of >= (int)m->tensors.size())
        return -1;
    const Tensor& src = m->tensors[of]->t;
    if (m->tensors[of]->alias_of >= 0 && !is_contiguous(src.layout)) {
        fail(TinyNN_ERROR_INVALID_LAYOUT, "model_add_view: a view of a strided view");
        return -1;
    }
    int id = add_tensor(m, name, nr_dim, dims, src.dtype.type_enum, src.dtype.param.scale);
    if (id < 0)
        return -1;
    Tensor& t = m->tensors[id]->t;
    for (int i = 0; i < nr_dim; ++i)
        t.layout.stride[i] = strides[i];
    long long lo, hi;
    const long long es = (long long)dtype_size(&t);
    if (view_span(t.layout, &lo, &hi) &&
        ((long long)offset_bytes + lo * es < 0 ||
         (long long)offset_bytes + (hi + 1) * es > (long long)tensor_bytes(src))) {
        fail(TinyNN_ERROR_OUT_OF_RANGE, "model_add_view: view leaves the %zu bytes of tensor %d",
             tensor_bytes(src), of);
        return -1;
    }
    m->tensors[id]->alias_of = of;
    m->tensors[id]->alias_offset = offset_bytes;
    return id;
}

static TinyNNStatus add_opr(
        Model* m, const MegccKernelDesc& desc, const char* symbol, const int* inputs, int nr_input,
        const int* outputs, int nr_output) {
    ModelOpr* o = new ModelOpr();
    o->desc = desc;
    o->symbol = symbol;
    memset(&o->ws, 0, sizeof(o->ws));
    const int idx = (int)m->oprs.size();
    for (int i = 0; i < nr_input; ++i) {
        if (inputs[i] < 0 || inputs[i] >= (int)m->tensors.size()) {
            delete o;
            return fail(TinyNN_ERROR_OUT_OF_RANGE, "model_add_opr: input id %d", inputs[i]);
        }
        o->in.push_back(inputs[i]);
        ModelTensor* t = m->tensors[root_of(m, inputs[i])];
        t->last = std::max(t->last, idx);
    }
    for (int i = 0; i < nr_output; ++i) {
        if (outputs[i] < 0 || outputs[i] >= (int)m->tensors.size()) {
            delete o;
            return fail(TinyNN_ERROR_OUT_OF_RANGE, "model_add_opr: output id %d", outputs[i]);
        }
        o->out.push_back(outputs[i]);
        ModelTensor* t = m->tensors[root_of(m, outputs[i])];
        if (t->def < 0)
            t->def = idx;
        t->last = std::max(t->last, idx);
    }
    m->oprs.push_back(o);
    return TinyNN_SUCCESS;
}

TinyNNStatus megcc_gfx950_model_add_opr(
        void* model, const char* symbol, const int* inputs, int nr_input, const int* outputs,
        int nr_output) {
    Model* m = (Model*)model;
    MG_REQUIRE(m && symbol && inputs && outputs && !m->finalized, TinyNN_ERROR_NULL_PTR,
               "model_add_opr: bad argument");
    MegccKernelDesc desc;
    TinyNNStatus st = megcc_gfx950_parse_symbol(symbol, &desc);
    if (st != TinyNN_SUCCESS)
        return st;
    return add_opr(m, desc, symbol, inputs, nr_input, outputs, nr_output);
}

TinyNNStatus megcc_gfx950_model_add_opr_desc(
        void* model, const MegccKernelDesc* desc, const char* name, const int* inputs, int nr_input,
        const int* outputs, int nr_output) {
    Model* m = (Model*)model;
    MG_REQUIRE(m && desc && name && inputs && outputs && !m->finalized, TinyNN_ERROR_NULL_PTR,
               "model_add_opr_desc: bad argument");
    MG_REQUIRE(desc->kind >= MEGCC_KERN_CONV && desc->kind <= MEGCC_KERN_SOFTMAX,
               TinyNN_ERROR_OUT_OF_RANGE, "model_add_opr_desc: kind %d", (int)desc->kind);
    return add_opr(m, *desc, name, inputs, nr_input, outputs, nr_output);
}

TinyNNStatus megcc_gfx950_model_mark_io(void* model, int tensor, int is_output) {
    Model* m = (Model*)model;
    MG_REQUIRE(m && tensor >= 0 && tensor < (int)m->tensors.size(), TinyNN_ERROR_OUT_OF_RANGE,
               "model_mark_io: tensor id");
    ModelTensor* t = m->tensors[root_of(m, tensor)];
    if (is_output) {
        t->is_output = true;
    } else {
        t->is_input = true;
        t->def = 0;  // staged before the first opr
        if (t->last < 0)
            t->last = 0;
    }
    return TinyNN_SUCCESS;
}

// parse_model + init_model_weights + init_model_memory of the TinyNN runtime
TinyNNStatus megcc_gfx950_model_finalize(void* model) {
    Model* m = (Model*)model;
    MG_REQUIRE(m && !m->finalized, TinyNN_ERROR_NULL_PTR, "model_finalize: bad model");
    for (auto* t : m->tensors)
        if (t->is_input && t->def != 0)
            t->def = 0;
    // (planned twice: the arena of the operators as they are says how many bytes the tail's tensors
    //  may get for themselves - 128 MB or 85 % of that arena, whichever is more: the balanced tail of a
    //  MobileNetV1 needs about that at every batch, and more only cost cache reuse)
    m->tail_opr_begin = -1;
    MG_REQUIRE(plan_memory(m), TinyNN_ERROR_INVALID_LAYOUT,
               "model_finalize: memory plan");
    choose_tail(m, std::max((size_t)128 << 20, (size_t)(0.85 * (double)m->arena_bytes)));
    MG_REQUIRE(plan_memory(m), TinyNN_ERROR_INVALID_LAYOUT,
               "model_finalize: memory plan (alignment %zu)", (size_t)m->dev.alignment);
    m->arena = m->dev.malloc(m->arena_bytes ? m->arena_bytes : 1);
    MG_REQUIRE(m->arena, TinyNN_ERROR_MEMORY_MALLOC, "model_finalize: arena of %zu bytes",
               m->arena_bytes);
    for (auto* t : m->tensors) {
        if (t->is_weight || t->alias_of >= 0)
            continue;
        if (t->is_input) {
            // user memory in the TinyNN runtime (runtime/src/init.c:456-460); here a device
            // buffer of its own that set_input fills
            t->owned = m->dev.malloc(t->t.size ? t->t.size : 1);
            MG_REQUIRE(t->owned, TinyNN_ERROR_MEMORY_MALLOC, "model_finalize: input of %zu bytes",
                       (size_t)t->t.size);
            t->t.ptr = t->owned;
        } else {
            t->t.ptr = (char*)m->arena + t->t.offset;
        }
    }
    for (size_t i = 0; i < m->tensors.size(); ++i)
        if (m->tensors[i]->alias_of >= 0) {
            // a chain of views adds up its offsets (output->ptr = input->ptr + offset,
            // runtime/src/vm/memforward.c:43-53)
            size_t shift = 0;
            int id = (int)i;
            while (m->tensors[id]->alias_of >= 0) {
                shift += m->tensors[id]->alias_offset;
                id = m->tensors[id]->alias_of;
            }
            const Tensor& r = m->tensors[id]->t;
            m->tensors[i]->t.ptr = (char*)r.ptr + shift;
            m->tensors[i]->t.offset = r.offset + shift;
        }
    for (auto* o : m->oprs) {
        for (int id : o->in)
            o->in_ptrs.push_back(&m->tensors[id]->t);
        for (int id : o->out)
            o->out_ptrs.push_back(&m->tensors[id]->t);
        // workspace size, asked with the original weights like the compiler does
        // (the VM shares one workspace region between operators)
        {
            size_t bytes = 0;
            TinyNNStatus wst = megcc_gfx950_call_workspace(
                    &o->desc, o->in_ptrs.data(), (int)o->in_ptrs.size(), 1, &bytes);
            if (wst != TinyNN_SUCCESS)
                return wst;
            o->ws.size = bytes;
            if (bytes > m->workspace_bytes)
                m->workspace_bytes = bytes;
        }
        // three-phase init (runtime/src/init.c:94-131)
        int n = 0;
        TinyNNStatus st = megcc_gfx950_call_init(
                &o->desc, o->in_ptrs.data(), (int)o->in_ptrs.size(), nullptr, &n, &m->opt);
        if (st != TinyNN_SUCCESS)
            return st;
        MG_REQUIRE(n <= 1, TinyNN_ERROR_NO_IMPLEMENT, "model_finalize: %d processed weights", n);
        if (n == 1) {
            memset(&o->processed, 0, sizeof(Tensor));
            st = megcc_gfx950_call_init(
                    &o->desc, o->in_ptrs.data(), (int)o->in_ptrs.size(), &o->processed, nullptr,
                    &m->opt);
            if (st != TinyNN_SUCCESS)
                return st;
            size_t bytes = tensor_bytes(o->processed);
            o->processed_mem = m->dev.malloc(bytes);
            MG_REQUIRE(o->processed_mem, TinyNN_ERROR_MEMORY_MALLOC,
                       "model_finalize: processed weight of %zu bytes", bytes);
            o->processed.ptr = o->processed_mem;
            o->processed.size = bytes;
            o->processed.is_weight = 1;
            st = megcc_gfx950_call_init(
                    &o->desc, o->in_ptrs.data(), (int)o->in_ptrs.size(), &o->processed, &n,
                    &m->opt);
            if (st != TinyNN_SUCCESS)
                return st;
            // the processed weight replaces the input with the same name (init.c:60-91)
            for (size_t j = 0; j < o->in_ptrs.size(); ++j)
                if (o->in_ptrs[j]->name == o->processed.name) {
                    o->in_ptrs[j] = &o->processed;
                    o->has_processed = true;
                    break;
                }
            MG_REQUIRE(o->has_processed, TinyNN_ERROR_NO_FOUND,
                       "model_finalize: %s: processed weight matches no input", o->symbol.c_str());
        }
    }
    if (m->workspace_bytes) {
        m->workspace = m->dev.malloc(m->workspace_bytes);
        MG_REQUIRE(m->workspace, TinyNN_ERROR_MEMORY_MALLOC, "model_finalize: workspace of %zu bytes",
                   m->workspace_bytes);
        for (auto* o : m->oprs)
            o->ws.ptr = o->ws.size ? m->workspace : nullptr;
    }
    build_schedule(m);
    setup_tail(m);
    // The balance of measured kernel times is only a starting point: one kernel more or less on the
    // tail moves MobileNetV1 batch 64 by 3 %. The boundary and its three neighbours on either side are
    // timed as whole forwards and the best one kept.
    auto tune_tail = [&]() -> float {
        if (m->tail_begin < 0)
            return -1.f;
        int best_tb = m->tail_begin;
        float best = time_forwards(m);
        const int tb0 = best_tb;
        for (int cand : {tb0 + 1, tb0 - 1, tb0 + 2, tb0 - 2, tb0 + 3, tb0 - 3}) {
            reset_tail(m);
            setup_tail(m, cand);
            if (m->tail_begin != cand)
                continue;
            const float t = time_forwards(m);
            if (t > 0.f && (best <= 0.f || t < best)) {
                best = t;
                best_tb = cand;
            }
        }
        if (m->tail_begin != best_tb) {
            reset_tail(m);
            setup_tail(m, best_tb);
        }
        return best;
    };
    const float with = tune_tail();
    // Pointwise -> depthwise pairs were judged one by one, kernel behind kernel on one stream. With
    // two streams the launch floors they save are hidden anyway and their one-workgroup-per-image
    // form fills the chip worse (MobileNetV1 batch 64: 248 k img/s with the pairs as one kernel, 263 k
    // as two; batch 32 the other way round): the whole forward is timed both ways and the faster
    // schedule kept.
    bool has_pair = false;
    for (const ModelOpr* o : m->schedule)
        has_pair = has_pair || o->desc.kind == MEGCC_KERN_PW_DW;
    if (with > 0.f && has_pair && !options().fuse_pwdw) {
        const std::vector<ModelOpr*> fused_schedule = m->schedule;
        const int fused_tb = m->tail_begin;
        reset_tail(m);
        build_schedule(m, false);
        setup_tail(m);
        const float without = tune_tail();
        if (!(without > 0.f && without < 0.98f * with)) {
            reset_tail(m);
            m->schedule = fused_schedule;
            setup_tail(m, fused_tb);
        }
    }
    m->finalized = true;
    return megcc_gfx950_wait();
}

// The compiler's static memory plan for a model built in memory: what a `.tiny` file carries as
// Tensor.offset and DeviceModel.tensor_memory (runtime/schema/model.fbs:63-124, consumed by
// runtime/src/init.c:437-487). finalize() then uses these offsets instead of planning.
TinyNNStatus megcc_gfx950_model_set_plan(
        void* model, const size_t* offsets, int nr_tensor, size_t arena_bytes) {
    Model* m = (Model*)model;
    MG_REQUIRE(m && offsets && !m->finalized, TinyNN_ERROR_NULL_PTR, "model_set_plan: bad argument");
    MG_REQUIRE(nr_tensor == (int)m->tensors.size(), TinyNN_ERROR_OUT_OF_RANGE,
               "model_set_plan: %d offsets for %zu tensors", nr_tensor, m->tensors.size());
    for (int i = 0; i < nr_tensor; ++i) {
        ModelTensor* t = m->tensors[i];
        if (t->is_weight || t->is_input || t->alias_of >= 0)
            continue;
        MG_REQUIRE(offsets[i] % m->dev.alignment == 0 && offsets[i] <= arena_bytes &&
                           t->t.size <= arena_bytes - offsets[i],
                   TinyNN_ERROR_INVALID_LAYOUT,
                   "model_set_plan: tensor %d: %zu bytes at offset %zu of a %zu byte arena (alignment %zu)",
                   i, (size_t)t->t.size, offsets[i], arena_bytes, (size_t)m->dev.alignment);
    }
    for (int i = 0; i < nr_tensor; ++i)
        m->tensors[i]->t.offset = offsets[i];
    m->arena_bytes = arena_bytes;
    m->preplanned = true;
    return TinyNN_SUCCESS;
}

// What forward() does with the model: the number of kernels of its schedule (operator chains that
// run as one kernel count once), and how it launches them.
int megcc_gfx950_model_nr_kernel(void* model) {
    Model* m = (Model*)model;
    return m && m->finalized ? (int)m->schedule.size() : 0;
}

int megcc_gfx950_model_launch_mode(void* model, float* eager_ms, float* graph_ms) {
    Model* m = (Model*)model;
    if (!m)
        return 0;
    if (eager_ms)
        *eager_ms = m->eager_ms < 1e29f ? m->eager_ms : -1.f;
    if (graph_ms)
        *graph_ms = m->graph_ms < 1e29f ? m->graph_ms : -1.f;
    return m->graph_state;
}

size_t megcc_gfx950_model_arena_bytes(void* model) {
    return model ? ((Model*)model)->arena_bytes : 0;
}

void* megcc_gfx950_model_tensor_ptr(void* model, int tensor) {
    Model* m = (Model*)model;
    if (!m || tensor < 0 || tensor >= (int)m->tensors.size())
        return nullptr;
    return m->tensors[tensor]->t.ptr;
}

// LITE_reset_tensor_memory + the staging copy (runtime/src/lite/tensor.c:93-112)
TinyNNStatus megcc_gfx950_model_set_input(void* model, int tensor, const void* host, size_t bytes) {
    Model* m = (Model*)model;
    MG_REQUIRE(m && m->finalized && tensor >= 0 && tensor < (int)m->tensors.size(),
               TinyNN_ERROR_OUT_OF_RANGE, "model_set_input: bad tensor");
    Tensor& t = m->tensors[tensor]->t;
    MG_REQUIRE(bytes == tensor_bytes(t), TinyNN_ERROR_INVALID_LAYOUT,
               "model_set_input: %zu bytes given, tensor has %zu", bytes, tensor_bytes(t));
    if (m->tail_reads_input)
        join_tail(m);  // (the last forward's tail may still be reading a model input)
    return megcc_gfx950_memcpy_h2d(t.ptr, host, bytes);
}

TinyNNStatus megcc_gfx950_model_get_output(void* model, int tensor, void* host, size_t bytes) {
    Model* m = (Model*)model;
    MG_REQUIRE(m && m->finalized && tensor >= 0 && tensor < (int)m->tensors.size(),
               TinyNN_ERROR_OUT_OF_RANGE, "model_get_output: bad tensor");
    Tensor& t = m->tensors[tensor]->t;
    MG_REQUIRE(bytes == tensor_bytes(t), TinyNN_ERROR_INVALID_LAYOUT,
               "model_get_output: %zu bytes asked, tensor has %zu", bytes, tensor_bytes(t));
    join_tail(m);
    return megcc_gfx950_memcpy_d2h(host, t.ptr, bytes);
}

// The copy is enqueued behind the forward that produced the tensor - on the tail stream when the last
// forward left its tail there - and the host does not wait: a caller that enqueues forward i, this
// copy, the next input and forward i + 1 keeps the overlap of forward i's tail with forward i + 1's
// head, which the blocking get_output cannot (the host would not enqueue forward i + 1 before
// forward i is over). `host` should be pinned memory; the bytes are there after megcc_gfx950_wait().
TinyNNStatus megcc_gfx950_model_get_output_async(void* model, int tensor, void* host, size_t bytes) {
    Model* m = (Model*)model;
    MG_REQUIRE(m && m->finalized && host && tensor >= 0 && tensor < (int)m->tensors.size(),
               TinyNN_ERROR_OUT_OF_RANGE, "model_get_output_async: bad argument");
    Tensor& t = m->tensors[tensor]->t;
    MG_REQUIRE(bytes == tensor_bytes(t), TinyNN_ERROR_INVALID_LAYOUT,
               "model_get_output_async: %zu bytes asked, tensor has %zu", bytes, tensor_bytes(t));
    // a tensor the tail writes: behind the tail, on its stream (the next forward's tail follows the
    // copy there); any other: on the library stream, between this forward's head and the next one's
    bool by_tail = false;
    for (const Tensor* w : m->tail_writes)
        by_tail = by_tail || shares_bytes(*w, t);
    hipStream_t s = m->tail_pending && by_tail ? m->tail_stream : main_stream();
    hipError_t e = hipMemcpyAsync(host, t.ptr, bytes, hipMemcpyDeviceToHost, s);
    MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "model_get_output_async: %s", hipGetErrorString(e));
    return TinyNN_SUCCESS;
}

TinyNNStatus megcc_gfx950_model_forward(void* model) {
    Model* m = (Model*)model;
    MG_REQUIRE(m && m->finalized, TinyNN_ERROR_NULL_PTR, "model_forward: model not finalized");
    ++m->forwards;
    auto replay = [&]() -> TinyNNStatus {
        join_tail(m);  // (a plain-launch forward before this one may have left its tail on the second stream)
        hipError_t e = hipGraphLaunch(m->graph_exec, stream());
        MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "model_forward: graph launch: %s", hipGetErrorString(e));
        return TinyNN_SUCCESS;
    };
    if (m->graph_state == 1)
        return replay();
    if (m->graph_state == -1)
        return forward_eager(m, true);
    // ---- undecided: the first ten forwards (1: plain; 2, 3, 7, 8: timed plain launches; 4: the capture
    //      and its first replay; 5, 6, 9, 10: timed replays)
    // (schedules of fewer than 5 kernels stay eager without asking: the depthwise + pooling + addition
    //  chain as one kernel takes 7.6 us per forward eagerly, 16.2 us as a graph)
    if (options().no_graph || m->schedule.size() < 5) {
        m->graph_state = -1;
        return forward_eager(m);
    }
    if (m->forwards == 1)
        return forward_eager(m);
    if (!m->ev0 && (hipEventCreate(&m->ev0) != hipSuccess || hipEventCreate(&m->ev1) != hipSuccess)) {
        m->graph_state = -1;
        return forward_eager(m);
    }
    // Two consecutive forwards, an event behind the last operator of each; keeps the shortest cost
    // seen. The cost of a way of launching is what limits back-to-back forwards: the time from the end
    // of one forward to the end of the next on the device - under plain launches the second one's
    // first operators overlap the first one's last, which are on the second stream - or, when that
    // is longer, the time the host needs to enqueue a forward behind another (26 plain launches of a
    // batch-1 network take the host longer than the device takes to run them). The first forward of a
    // pair returns at once, the second one blocks until both are done.
    auto timed = [&](bool graph, bool second, float* best) -> TinyNNStatus {
        hipEvent_t done = second ? m->ev1 : m->ev0;
        const auto h0 = std::chrono::steady_clock::now();
        TinyNNStatus st;
        if (graph) {
            st = replay();
            (void)hipEventRecord(done, main_stream());
        } else {
            st = forward_eager(m, true, done);
        }
        const float host_ms = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - h0).count();
        if (!second)
            return st;
        float ms = 0.f;
        if (st == TinyNN_SUCCESS && hipEventSynchronize(m->ev1) == hipSuccess &&
            hipEventElapsedTime(&ms, m->ev0, m->ev1) == hipSuccess) {
            const float cost = ms > host_ms ? ms : host_ms;
            if (cost < *best)
                *best = cost;
        }
        return st;
    };
    if (m->forwards <= 3 || (m->graph_exec && (m->forwards == 7 || m->forwards == 8)))
        return timed(false, m->forwards == 3 || m->forwards == 8, &m->eager_ms);
    if (m->forwards == 4) {
        join_tail(m);  // (before the capture begins: the wait refers to an event outside of it)
        if (hipStreamBeginCapture(stream(), hipStreamCaptureModeThreadLocal) == hipSuccess) {
            TinyNNStatus st = forward_eager(m);
            hipGraph_t g = nullptr;
            hipError_t e = hipStreamEndCapture(stream(), &g);
            if (st == TinyNN_SUCCESS && e == hipSuccess && g &&
                hipGraphInstantiate(&m->graph_exec, g, nullptr, nullptr, 0) == hipSuccess) {
                m->graph = g;
                return replay();
            }
            if (g)
                (void)hipGraphDestroy(g);
            (void)hipGetLastError();  // a failed capture must not poison the eager path
            if (st != TinyNN_SUCCESS)
                return st;
        }
        m->graph_state = -1;
        return forward_eager(m);
    }
    TinyNNStatus st = timed(true, m->forwards == 6 || m->forwards == 10, &m->graph_ms);
    // (the shorter of two pairs each: a single sample of a 0.12 ms forward is off by several percent,
    //  which flipped the choice for batch-1 networks from run to run; a tie keeps the plain launches)
    if (m->forwards >= 10)
        m->graph_state = m->graph_ms < 0.98f * m->eager_ms ? 1 : -1;
    return st;
}

// Kernels of one forward that go to the second stream under plain launches (0: none).
int megcc_gfx950_model_nr_tail_kernel(void* model) {
    Model* m = (Model*)model;
    return m && m->finalized && m->tail_begin >= 0 ? (int)m->schedule.size() - m->tail_begin : 0;
}

// Orders the library stream behind everything the model's forwards have launched (the last
// operators of a forward may run on a second stream; see Model::tail_begin).
TinyNNStatus megcc_gfx950_model_join(void* model) {
    Model* m = (Model*)model;
    MG_REQUIRE(m && m->finalized, TinyNN_ERROR_NULL_PTR, "model_join: model not finalized");
    join_tail(m);
    return TinyNN_SUCCESS;
}

int megcc_gfx950_model_nr_opr(void* model) {
    return model ? (int)((Model*)model)->oprs.size() : 0;
}

// Runs a single instruction (per-layer timing and tensor dumps, the TINYNN_PROFILE_KERNEL /
// TINYNN_DUMP_TENSOR hooks of network.c:187-224)
TinyNNStatus megcc_gfx950_model_run_opr(void* model, int index) {
    Model* m = (Model*)model;
    MG_REQUIRE(m && m->finalized && index >= 0 && index < (int)m->oprs.size(),
               TinyNN_ERROR_OUT_OF_RANGE, "model_run_opr: index %d", index);
    ModelOpr* o = m->oprs[index];
    join_tail(m);
    return megcc_gfx950_call(
            &o->desc, o->in_ptrs.data(), (int)o->in_ptrs.size(), o->out_ptrs.data(),
            (int)o->out_ptrs.size(), &o->ws, &m->opt);
}

// The static memory plan on its own, for a caller that has the lifetimes (the compiler side, or a
// loader that wants to check the offsets stored in a model file).
TinyNNStatus megcc_gfx950_plan_memory(
        size_t nr_interval, const size_t* begin, const size_t* end, const size_t* size,
        size_t alignment, size_t* offset, size_t* arena_bytes, size_t* lower_bound) {
    MG_REQUIRE(nr_interval == 0 || (begin && end && size && offset), TinyNN_ERROR_NULL_PTR,
               "plan_memory: null array");
    MG_REQUIRE(arena_bytes, TinyNN_ERROR_NULL_PTR, "plan_memory: null arena_bytes");
    std::vector<MemInterval> intervals(nr_interval);
    for (size_t i = 0; i < nr_interval; ++i)
        intervals[i] = MemInterval{begin[i], end[i], size[i]};
    std::vector<size_t> offsets;
    MG_REQUIRE(plan_memory_pushdown(intervals, alignment, &offsets, arena_bytes, lower_bound),
               TinyNN_ERROR_INVALID_LAYOUT,
               "plan_memory: alignment %zu is not a power of two, or an interval is empty",
               alignment);
    for (size_t i = 0; i < nr_interval; ++i)
        offset[i] = offsets[i];
    return TinyNN_SUCCESS;
}

// ---- `.tiny` model files ------------------------------------------------------------------------

TinyNNStatus megcc_gfx950_tiny_describe(
        const void* buffer, size_t size, char* text, size_t capacity, size_t* needed) {
    tiny::ModelInfo info;
    std::string err;
    MG_REQUIRE(tiny::read_model(buffer, size, &info, &err), TinyNN_ERROR_MODEL_PARSE,
               "tiny_describe: %s", err.c_str());
    const std::string s = tiny::describe(info);
    if (needed)
        *needed = s.size() + 1;
    if (text && capacity) {
        const size_t n = std::min(capacity - 1, s.size());
        memcpy(text, s.data(), n);
        text[n] = 0;
    }
    return TinyNN_SUCCESS;
}

namespace {

float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000) << 16;
    uint32_t e = (h >> 10) & 31, mant = h & 1023, bits;
    if (e == 0) {
        if (mant == 0) {
            bits = sign;
        } else {  // subnormal: renormalise
            int shift = 0;
            while (!(mant & 1024)) {
                mant <<= 1;
                ++shift;
            }
            bits = sign | ((uint32_t)(113 - shift) << 23) | ((mant & 1023) << 13);
        }
    } else if (e == 31) {
        bits = sign | 0x7f800000u | (mant << 13);
    } else {
        bits = sign | ((e + 112) << 23) | (mant << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

// model tensor from a file entry; false (with the error set) when the entry cannot be used
bool tensor_from_file(
        Model* m, const tiny::DType& dt, const tiny::Layout& l, const std::string& name,
        int* id) {
    const int nd = (int)l.dims.size();
    if (nd < 1 || nd > MAX_DIM || l.stride.size() != l.dims.size()) {
        fail(TinyNN_ERROR_MODEL_PARSE, "model_load: tensor %s has %d dims, %zu strides",
             name.c_str(), nd, l.stride.size());
        return false;
    }
    uint32_t dims[MAX_DIM];
    for (int i = 0; i < nd; ++i) {
        if (l.dims[i] < 0) {
            fail(TinyNN_ERROR_MODEL_PARSE, "model_load: tensor %s: negative dim", name.c_str());
            return false;
        }
        dims[i] = (uint32_t)l.dims[i];
    }
    switch (dt.type) {
        case tiny::DT_Float32: case tiny::DT_Float16: case tiny::DT_Int32: case tiny::DT_Int8:
        case tiny::DT_Int16: case tiny::DT_Uint8: case tiny::DT_QInt8: case tiny::DT_QInt32:
        case tiny::DT_QUint8:
            break;
        default:
            fail(TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE, "model_load: tensor %s: dtype %d",
                 name.c_str(), dt.type);
            return false;
    }
    // the schema's enum values are the runtime's (runtime/src/parse.c:33-58)
    *id = add_tensor(m, name.c_str(), nd, dims, (TinyNNDType)dt.type,
                     dt.has_param ? dt.scale : 0.0f);
    if (*id < 0) {
        fail(TinyNN_ERROR_MODEL_PARSE, "model_load: tensor %s rejected", name.c_str());
        return false;
    }
    Tensor& t = m->tensors[*id]->t;
    t.dtype.param.zero_point = (uint8_t)dt.zero_point;
    for (int i = 0; i < nd; ++i)
        t.layout.stride[i] = l.stride[i];
    t.layout.format = (TinyNNFormat)l.format;
    return true;
}

TinyNNStatus load_into(Model* m, const tiny::ModelInfo& info) {
    // the device model compiled for this device if there is one, else the BARE_METAL one: its
    // instructions name the very kernels this library replaces
    const tiny::DeviceModelInfo* dm = nullptr;
    for (const auto& d : info.device_models)
        if (d.device == tiny::DEV_GFX950)
            dm = &d;
    if (!dm)
        for (const auto& d : info.device_models)
            if (d.device == tiny::DEV_BARE_METAL) {
                dm = &d;
                break;
            }
    MG_REQUIRE(dm, TinyNN_ERROR_NO_FOUND,
               "model_load: %zu device models, none for gfx950 or BARE_METAL",
               info.device_models.size());

    m->preplanned = true;
    m->arena_bytes = dm->tensor_memory;
    const int nt = (int)dm->tensors.size(), nw = (int)info.weights.size();
    for (int i = 0; i < nt; ++i) {
        const tiny::TensorInfo& ti = dm->tensors[i];
        MG_REQUIRE(!ti.dynamic, TinyNN_ERROR_NO_IMPLEMENT,
                   "model_load: tensor %d is dynamic (only static shapes run here)", i);
        char dflt[32];
        snprintf(dflt, sizeof(dflt), "tensor:%d", i);  // parse.c:121-127
        int id = -1;
        if (!tensor_from_file(m, ti.dtype, ti.layout, ti.name.empty() ? std::string(dflt) : ti.name, &id))
            return TinyNN_ERROR_MODEL_PARSE;
        ModelTensor* t = m->tensors[id];
        t->t.use_count = ti.use_count;
        MG_REQUIRE(ti.offset >= 0, TinyNN_ERROR_MODEL_PARSE, "model_load: tensor %d: offset", i);
        t->t.offset = (size_t)ti.offset;
    }
    for (int j = 0; j < nw; ++j) {
        const tiny::WeightInfo& wi = info.weights[j];
        int id = -1;
        if (!tensor_from_file(m, wi.dtype, wi.layout, wi.name, &id))
            return TinyNN_ERROR_MODEL_PARSE;
        ModelTensor* t = m->tensors[id];
        t->is_weight = true;
        t->t.is_weight = 1;
        t->t.use_count = wi.use_count;
        t->t.checksum = wi.checksum;
        const size_t bytes = t->t.size;
        std::vector<float> wide;
        const void* host = wi.data;
        if (wi.dtype.type == tiny::DT_Float32 && bytes && wi.data_bytes == bytes / 2) {
            // fp32 weight stored as fp16 (parse.c:232-263)
            wide.resize(bytes / 4);
            for (size_t k = 0; k < wide.size(); ++k) {
                uint16_t h;
                memcpy(&h, wi.data + 2 * k, 2);
                wide[k] = half_to_float(h);
            }
            host = wide.data();
        } else {
            MG_REQUIRE(wi.data_bytes == bytes, TinyNN_ERROR_MODEL_PARSE,
                       "model_load: weight %s holds %zu bytes, its layout needs %zu",
                       wi.name.c_str(), wi.data_bytes, bytes);
        }
        t->owned = m->dev.malloc(bytes ? bytes : 1);
        MG_REQUIRE(t->owned, TinyNN_ERROR_MEMORY_MALLOC, "model_load: weight of %zu bytes", bytes);
        t->t.ptr = t->owned;
        if (bytes) {
            TinyNNStatus st = megcc_gfx950_memcpy_h2d(t->owned, host, bytes);
            if (st != TinyNN_SUCCESS)
                return st;
        }
    }

    for (int idx : dm->inputs) {
        MG_REQUIRE(idx >= 0 && idx < nt, TinyNN_ERROR_MODEL_PARSE, "model_load: input index %d", idx);
        TinyNNStatus st = megcc_gfx950_model_mark_io(m, idx, 0);
        if (st != TinyNN_SUCCESS)
            return st;
        m->tensors[idx]->t.is_input = 1;
    }
    for (int idx : dm->outputs) {
        MG_REQUIRE(idx >= 0 && idx < nt, TinyNN_ERROR_MODEL_PARSE, "model_load: output index %d", idx);
        megcc_gfx950_model_mark_io(m, idx, 1);
    }

    for (size_t k = 0; k < dm->instructions.size(); ++k) {
        const tiny::Instruction& in = dm->instructions[k];
        if (in.kind == tiny::INST_Opr) {
            MG_REQUIRE(in.input_types.size() == in.inputs.size(), TinyNN_ERROR_MODEL_PARSE,
                       "model_load: instruction %zu: %zu inputs, %zu input types", k,
                       in.inputs.size(), in.input_types.size());
            std::vector<int> ins, outs;
            for (size_t i = 0; i < in.inputs.size(); ++i) {
                const bool w = in.input_types[i] == tiny::TT_WEIGHT;
                const int idx = in.inputs[i];
                MG_REQUIRE(idx >= 0 && idx < (w ? nw : nt), TinyNN_ERROR_MODEL_PARSE,
                           "model_load: instruction %zu: input index %d", k, idx);
                ins.push_back(w ? nt + idx : idx);
            }
            for (int idx : in.outputs) {
                MG_REQUIRE(idx >= 0 && idx < nt, TinyNN_ERROR_MODEL_PARSE,
                           "model_load: instruction %zu: output index %d", k, idx);
                outs.push_back(idx);
            }
            TinyNNStatus st = megcc_gfx950_model_add_opr(
                    m, in.type.c_str(), ins.data(), (int)ins.size(), outs.data(), (int)outs.size());
            if (st != TinyNN_SUCCESS)
                return st == TinyNN_ERROR_NO_FOUND
                             ? fail(TinyNN_ERROR_NO_FOUND,
                                    "model_load: instruction %zu: no gfx950 kernel for %s", k,
                                    in.type.c_str())
                             : st;
        } else if (in.kind == tiny::INST_MemForward) {
            const int src = in.fwd_input, dst = in.fwd_output;
            MG_REQUIRE(src >= 0 && src < nt && dst >= 0 && dst < nt && src != dst,
                       TinyNN_ERROR_MODEL_PARSE, "model_load: instruction %zu: MemForward %d -> %d",
                       k, src, dst);
            ModelTensor* o = m->tensors[dst];
            MG_REQUIRE(o->alias_of < 0 && o->def < 0, TinyNN_ERROR_MODEL_PARSE,
                       "model_load: instruction %zu: tensor %d already has memory", k, dst);
            MG_REQUIRE(in.fwd_offset >= 0, TinyNN_ERROR_MODEL_PARSE,
                       "model_load: instruction %zu: negative MemForward offset", k);
            for (int id = src, hops = 0; id >= 0; id = m->tensors[id]->alias_of)
                MG_REQUIRE(id != dst && ++hops <= nt, TinyNN_ERROR_MODEL_PARSE,
                           "model_load: instruction %zu: MemForward cycle", k);
            o->alias_of = src;
            o->alias_offset = (size_t)in.fwd_offset;
        } else {
            return fail(TinyNN_ERROR_UNSUPPORTED_INSTRUCTION_TYPE,
                        "model_load: instruction %zu has type %d; this runtime executes Opr and "
                        "MemForward", k, in.kind);
        }
    }

    // every byte a kernel may touch lies inside the arena (or inside the tensor a view points at);
    // only views may be strided
    for (int i = 0; i < nt; ++i) {
        ModelTensor* t = m->tensors[i];
        if (t->alias_of >= 0) {
            long long shift = 0;
            int id = i, hops = 0;
            while (m->tensors[id]->alias_of >= 0) {
                shift += (long long)m->tensors[id]->alias_offset;
                id = m->tensors[id]->alias_of;
                MG_REQUIRE(++hops <= nt, TinyNN_ERROR_MODEL_PARSE, "model_load: MemForward cycle");
            }
            long long lo, hi;
            if (!view_span(t->t.layout, &lo, &hi))
                continue;  // no elements
            const long long es = (long long)dtype_size(&t->t);
            MG_REQUIRE(shift + lo * es >= 0 &&
                               shift + (hi + 1) * es <= (long long)m->tensors[id]->t.size,
                       TinyNN_ERROR_MODEL_PARSE,
                       "model_load: tensor %d views bytes %lld..%lld of tensor %d (%zu bytes)", i,
                       shift + lo * es, shift + (hi + 1) * es, id, (size_t)m->tensors[id]->t.size);
        } else {
            MG_REQUIRE(is_contiguous(t->t.layout), TinyNN_ERROR_MODEL_PARSE,
                       "model_load: tensor %d owns memory but is not dense", i);
            if (!t->is_input)
                MG_REQUIRE(t->t.offset + t->t.size <= m->arena_bytes, TinyNN_ERROR_MODEL_PARSE,
                           "model_load: tensor %d ends at byte %zu of a %zu byte arena", i,
                           (size_t)(t->t.offset + t->t.size), m->arena_bytes);
        }
    }
    return megcc_gfx950_model_finalize(m);
}

}  // namespace

// parse_model + init_model_weights + init_model_memory (runtime/src/parse.c:423-560,
// runtime/src/init.c) for this device. Tensor ids of the returned model: the file's tensor_pool
// index; weight j of the weight_pool is id nr_tensor + j.
TinyNNStatus megcc_gfx950_model_load(const void* buffer, size_t size, void** model) {
    MG_REQUIRE(model, TinyNN_ERROR_NULL_PTR, "model_load: null result pointer");
    *model = nullptr;
    tiny::ModelInfo info;
    std::string err;
    MG_REQUIRE(tiny::read_model(buffer, size, &info, &err), TinyNN_ERROR_MODEL_PARSE,
               "model_load: %s", err.c_str());
    Model* m = (Model*)megcc_gfx950_model_create();
    MG_REQUIRE(m, TinyNN_ERROR_RUNTIME, "model_load: no device");
    TinyNNStatus st = load_into(m, info);
    if (st != TinyNN_SUCCESS) {
        megcc_gfx950_model_destroy(m);
        return st;
    }
    *model = m;
    return TinyNN_SUCCESS;
}

}  // extern "C"
