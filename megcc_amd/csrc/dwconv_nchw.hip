// qsi8 channel-wise (depthwise GROUP) 3x3 convolution, pad 1, stride 1 or 2, on plain NCHW tensors
// (kernel_conv2d_3x3_NCHW_GROUP_p1x1_s?x?_d1x1_qsi8qsi8qsi32qsi8_bias[_ACT]): tensor [N,C,H,W],
// filter [C,1,1,3,3], one plane per channel (BareMetal/ConvKernel.cpp:62-64,305-344).
//
// In NCHW the bytes of a row are consecutive pixels of ONE channel, which is exactly what
// v_dot4_i32_i8 wants: the three horizontal taps of an output pixel are three neighbouring bytes.
// A thread makes groups of 4 neighbouring output pixels of a row (one dword store each). Per input
// row and group it uses the aligned dwords A (the 4 pixels left of the group), B (the group) and C
// (the 4 pixels right of it) - with stride 2 the group is 8 input pixels wide and A, B, C are the
// dword left of it and its two dwords - and builds the windows with two v_alignbyte:
//   stride 1: (A3 B0 B1 B2) serves outputs 0 and 1, (B1 B2 B3 C0) outputs 2 and 3,
//   stride 2: (A3 B0 B1 B2) output 0, B output 1, (B3 C0 C1 C2) output 2, C output 3,
// where the even use meets the weights (w0, w1, w2, 0) and the odd one the same weights moved up a
// byte, (0, w0, w1, w2). Rows are a multiple of 4 pixels, so an aligned dword never straddles a
// row: the dword left of the first group and right of the last one, and rows above / below the
// image, are loaded with an out-of-range buffer offset and read as zero - the padding costs no
// instruction. Any channel count (the NCHW44 detour needs multiples of 4).
// Accumulators start from the bias; exact requantisation by threshold table (epilogue.h).
#include "common.h"
#include "conv_geom.h"
#include "epilogue.h"
#include "fastdiv.h"

namespace mg {

struct DwNchwParams {
    const int8_t* src;
    const int8_t* flt;
    const int32_t* bias;  // or nullptr
    int8_t* dst;
    int src_bytes, dst_bytes, flt_bytes;
    int c, ih, iw, oh, ow;
    int ogn;    // column groups (G * 4 output pixels) per row
    int ohn;    // row groups (R output rows) per plane
    int total;  // threads: planes * ohn * ogn
    int act;
    float s_src, s_flt, s_dst, cf;
    float aff_c, aff_d;  // requantisation by one fused multiply-add (epilogue.h); aff_d == 0: table
    FastDiv d_ogn, d_oh, d_c;  // by ogn, ohn, c
    RequantTable table;
};

// G: groups of 4 output pixels per thread and row; R: output rows per thread. One thread per output
// dword spent four fifths of its instructions on index arithmetic, offsets and the table set-up
// (37 vector instructions per output, 31.7 us for N=64 C=32 112x112): 2 x 2 shares them between 16
// outputs and the input rows between two output rows.
template <int S, int ACT, int G, int R>
__global__ void __launch_bounds__(256) dwconv_nchw_3x3_kernel(DwNchwParams q) {
    constexpr int ND = S == 1 ? G + 2 : 2 * G + 1;  // dwords per input row: D[-1] .. D[ND - 2]
    constexpr int IR = (R - 1) * S + 3;             // input rows
    __shared__ int tbl[REQUANT_TABLE_ENTRIES];
    if (ACT >= 0) {
        tbl[threadIdx.x] = q.table.t[threadIdx.x];
        __syncthreads();
    }
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= q.total)
        return;
    // i = (plane * row groups + row group) * column groups + column group
    const int r1 = fdiv(i, q.d_ogn), og = i - r1 * q.ogn;
    const int plane = fdiv(r1, q.d_oh), oy = (r1 - plane * q.ohn) * R;
    const int ch = plane - fdiv(plane, q.d_c) * q.c;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)q.src, 0, q.src_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rf = __builtin_amdgcn_make_buffer_rsrc((void*)q.flt, 0, q.flt_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc((void*)q.dst, 0, q.dst_bytes, 0x00020000);
    const int OOB = (int)0x80000000u;
    // filter rows as (w0, w1, w2, 0): dword loads from byte offsets 9 ch, 9 ch + 3 and, for the last
    // row, 9 ch + 5 shifted down a byte, so that no load leaves the 9 bytes of the channel
    unsigned wq[3], ws[3];
    wq[0] = __builtin_amdgcn_raw_buffer_load_b32(rf, ch * 9, 0, 0) & 0x00ffffffu;
    wq[1] = __builtin_amdgcn_raw_buffer_load_b32(rf, ch * 9 + 3, 0, 0) & 0x00ffffffu;
    wq[2] = __builtin_amdgcn_raw_buffer_load_b32(rf, ch * 9 + 5, 0, 0) >> 8;
#pragma unroll
    for (int fh = 0; fh < 3; ++fh)
        ws[fh] = wq[fh] << 8;
    const int b = q.bias ? q.bias[ch] : 0;
    int acc[R][G * 4];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int e = 0; e < G * 4; ++e)
            acc[r][e] = b;
    const int xb = og * (G * 4 * S);  // first input pixel of D[0]
    bool col_ok[ND];                  // dword k - 1 lies inside the row
#pragma unroll
    for (int k = 0; k < ND; ++k)
        col_ok[k] = (unsigned)(xb + 4 * (k - 1)) < (unsigned)q.iw;
    const int plane_off = plane * q.ih * q.iw + xb;
#pragma unroll
    for (int ir = 0; ir < IR; ++ir) {
        const int iy = oy * S - 1 + ir;
        const bool row_ok = (unsigned)iy < (unsigned)q.ih;
        const int off = plane_off + __mul24(iy, q.iw);
        unsigned D[ND];
#pragma unroll
        for (int k = 0; k < ND; ++k)
            D[k] = __builtin_amdgcn_raw_buffer_load_b32(rs, row_ok && col_ok[k] ? off + 4 * (k - 1) : OOB, 0, 0);
        // the dwords whose bytes 0..2 (even outputs) or 1..3 (odd outputs) are the windows
        unsigned w[G * 4];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if (S == 1) {
                w[4 * g] = w[4 * g + 1] = __builtin_amdgcn_alignbyte(D[g + 1], D[g], 3);      // x-1 .. x+2
                w[4 * g + 2] = w[4 * g + 3] = __builtin_amdgcn_alignbyte(D[g + 2], D[g + 1], 1);  // x+1 .. x+4
            } else {
                w[4 * g] = __builtin_amdgcn_alignbyte(D[2 * g + 1], D[2 * g], 3);      // 2x-1 2x 2x+1
                w[4 * g + 1] = D[2 * g + 1];                                           // . 2x+1 2x+2 2x+3
                w[4 * g + 2] = __builtin_amdgcn_alignbyte(D[2 * g + 2], D[2 * g + 1], 3);  // 2x+3 2x+4 2x+5
                w[4 * g + 3] = D[2 * g + 2];                                           // . 2x+5 2x+6 2x+7
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int fh = ir - r * S;
            if (fh < 0 || fh > 2)
                continue;
#pragma unroll
            for (int e = 0; e < G * 4; ++e)
                acc[r][e] = __builtin_amdgcn_sdot4((int)w[e], (int)((e & 1) ? ws[fh] : wq[fh]), acc[r][e], false);
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (oy + r >= q.oh)
            break;
        int o[G * 4];
        if (ACT < 0) {
#pragma unroll
            for (int e = 0; e < G * 4; ++e)
                o[e] = requant_conv_rt(q.act, acc[r][e], q.s_src, q.s_flt, q.s_dst);
        } else if (q.aff_d != 0.f) {  // (uniform)
#pragma unroll
            for (int e = 0; e < G * 4; ++e)
                o[e] = requant_conv_affine<(ACT == MEGCC_NONLINE_RELU ? ACT : 0)>(acc[r][e], q.aff_c, q.aff_d);
        } else {
#pragma unroll
            for (int e = 0; e < G * 4; ++e)
                o[e] = requant_conv_table<(ACT < 0 ? 0 : ACT)>(acc[r][e], q.cf, tbl);
        }
        const int x0 = og * (G * 4);
        const int out = (plane * q.oh + oy + r) * q.ow + x0;
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if ((q.ow & 3) == 0) {
                __builtin_amdgcn_raw_buffer_store_b32(
                        pack4_perm(o[4 * g], o[4 * g + 1], o[4 * g + 2], o[4 * g + 3]), rd,
                        x0 + 4 * g < q.ow ? out + 4 * g : OOB, 0, 0);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (x0 + 4 * g + j < q.ow)
                        q.dst[out + 4 * g + j] = (int8_t)o[4 * g + j];
            }
        }
    }
}

bool dwconv_nchw_supported(const ConvGeom& g, const void* src, const void* dst) {
    return g.fmt == MEGCC_FMT_NCHW && g.groups > 1 && g.groups == g.ic && g.ic == g.oc && g.fh == 3 &&
           g.fw == 3 && g.ph == 1 && g.pw == 1 && g.dh == 1 && g.dw == 1 && g.sh == g.sw &&
           (g.sh == 1 || g.sh == 2) && (g.iw & 3) == 0 && ((uintptr_t)src & 3) == 0 &&
           ((uintptr_t)dst & 3) == 0 && (long)g.n * g.ic * g.ih * g.iw < (1L << 31) &&
           (long)g.n * g.oc * g.oh * g.ow < (1L << 31) && (long)g.ih * g.iw < (1L << 24) &&
           (long)g.ic * 9 < (1L << 31);
}

TinyNNStatus dwconv_nchw_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst) {
    DwNchwParams q = {};
    q.src = (const int8_t*)src;
    q.flt = (const int8_t*)flt;
    q.bias = (const int32_t*)bias;
    q.dst = (int8_t*)dst;
    q.src_bytes = (int)((long)g.n * g.ic * g.ih * g.iw);
    q.dst_bytes = (int)((long)g.n * g.oc * g.oh * g.ow);
    q.flt_bytes = g.ic * 9;
    q.c = g.ic;
    q.ih = g.ih;
    q.iw = g.iw;
    q.oh = g.oh;
    q.ow = g.ow;
    constexpr int G = 2, R = 2;
    q.ogn = (g.ow + 4 * G - 1) / (4 * G);
    q.ohn = (g.oh + R - 1) / R;
    const long total = (long)g.n * g.ic * q.ohn * q.ogn;
    if (total == 0)
        return TinyNN_SUCCESS;
    q.total = (int)total;
    q.act = g.act;
    q.s_src = g.s_src;
    q.s_flt = g.s_flt;
    q.s_dst = g.s_dst;
    q.cf = make_requant_fast(g.s_src, g.s_flt, g.s_dst).c;
    q.d_ogn = make_fastdiv(q.ogn);
    q.d_oh = make_fastdiv(q.ohn);
    q.d_c = make_fastdiv(g.ic);
    const bool tab = (g.act == MEGCC_NONLINE_IDENTITY || g.act == MEGCC_NONLINE_RELU) &&
                     requant_table_ok(g.s_src, g.s_flt, g.s_dst);
    if (tab)
        q.table = requant_table_for(g.act, g.s_src, g.s_flt, g.s_dst);
    const int act = tab ? g.act : -1;
    const RequantAffine aff = requant_affine_pick(tab, g.act, g.s_src, g.s_flt, g.s_dst);
    q.aff_c = aff.c;
    q.aff_d = aff.d;
    void (*kern)(DwNchwParams);
#define MG_DWN_PICK(S_)                                                                         \
    (act == MEGCC_NONLINE_IDENTITY ? dwconv_nchw_3x3_kernel<S_, MEGCC_NONLINE_IDENTITY, G, R>    \
     : act == MEGCC_NONLINE_RELU   ? dwconv_nchw_3x3_kernel<S_, MEGCC_NONLINE_RELU, G, R>        \
                                   : dwconv_nchw_3x3_kernel<S_, -1, G, R>)
    kern = g.sh == 1 ? MG_DWN_PICK(1) : MG_DWN_PICK(2);
#undef MG_DWN_PICK
    hipLaunchKernelGGL(kern, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream(), q);
    return check_launch("dwconv_nchw_3x3");
}

}  // namespace mg
