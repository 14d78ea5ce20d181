// conv on the HIP backend: the im2col composite of the reference (conv/im2col.rs:1-243) over
// rearrange and mat_mul.  y[n, m, hy, wy] = w[m, c, hk, wk] * x[n, c, h, w] + b[m]: the bias is
// broadcast into y by a rearrange, x is unfolded into a [n, c*hk*wk, hy*wy] matrix in workspace
// by a second rearrange (a 6-d strided copy), and one batched mat_mul with beta = 1 adds the
// product.  Padding is not supported, as in the reference.
#include "handle.hpp"

using namespace ophip;

namespace {

void sub(int code) {
    if (code != OPHIP_OK) throw Error{code, ophip_last_error()};
}

struct ConvMeta {
    uint64_t dt;
    size_t n, m, c, h, w, hy, wy, hk, wk;
};

// conv/args.rs:35-69
ConvMeta conv_meta(const ophip_conv_args &a) {
    expect_rank(a.y_layout, "y", 4);
    expect_rank(a.x_layout, "x", 4);
    expect_rank(a.w_layout, "w", 4);
    expect_rank(a.b_layout, "b", 1);
    ConvMeta r;
    r.dt = type_distinct({a.y_layout.dt, a.x_layout.dt, a.w_layout.dt, a.b_layout.dt});
    r.n = dim_distinct({a.x_layout.shape[0], a.y_layout.shape[0]});
    r.m = dim_distinct({a.w_layout.shape[0], a.y_layout.shape[1], a.b_layout.shape[0]});
    r.c = dim_distinct({a.x_layout.shape[1], a.w_layout.shape[1]});
    r.h = a.x_layout.shape[2];
    r.w = a.x_layout.shape[3];
    r.hy = a.y_layout.shape[2];
    r.wy = a.y_layout.shape[3];
    r.hk = a.w_layout.shape[2];
    r.wk = a.w_layout.shape[3];
    return r;
}

// ArrayLayout::merge_be over `count` adjacent dimensions: they fold into one when each stride is
// the next one times the next length (a dimension of length 1 folds with anything).
bool merge_be(const size_t *shape, const ptrdiff_t *strides, size_t count, size_t &len, ptrdiff_t &stride) {
    len = 1;
    stride = 0;
    bool have = false;
    ptrdiff_t prev_stride = 0;
    for (size_t i = count; i-- > 0;) {  // innermost first
        if (shape[i] == 1) continue;
        if (!have) {
            stride = strides[i];
            have = true;
        } else if (strides[i] != prev_stride) {
            return false;
        }
        prev_stride = strides[i] * (ptrdiff_t)shape[i];
        len *= shape[i];
    }
    return true;
}

void no_padding(const ophip_conv_args &a) {
    for (size_t p : a.pads)
        if (p != 0) throw args_not_support("non-zero padding for im2col is not supported");
}

}  // namespace

struct ophip_conv {
    ophip_device *dev;
    ophip_rearrange *rearrange = nullptr;
    ophip_mat_mul *mat_mul = nullptr;
    explicit ophip_conv(ophip_device *d) : dev(d) {
        ophip_device_retain(d);
        try {
            sub(ophip_rearrange_create(d, &rearrange));
            sub(ophip_mat_mul_create(d, &mat_mul));
        } catch (...) {
            release();
            throw;
        }
    }
    void release() {
        ophip_rearrange_destroy(rearrange);
        ophip_mat_mul_destroy(mat_mul);
        ophip_device_release(dev);
    }
    ~ophip_conv() { release(); }
    ophip_conv(const ophip_conv &) = delete;
    ophip_conv &operator=(const ophip_conv &) = delete;
};

extern "C" {

int ophip_conv_create(ophip_device *dev, ophip_conv **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        *out = new ophip_conv(dev);
    });
}
void ophip_conv_destroy(ophip_conv *op) { delete op; }

// Operator::scheme (conv/im2col.rs:42-83): the size of the unfolded x when every extent is
// known and it fits, else 0.
int ophip_conv_scheme(ophip_conv *, const ophip_conv_args *args, size_t max_ws, size_t *ws) {
    return guard([&] {
        if (ws) *ws = 0;
        if (!args) throw args_not_support("null argument");
        no_padding(*args);
        const ConvMeta r = conv_meta(*args);
        for (size_t v : {r.n, r.c, r.hk, r.wk, r.hy, r.wy})
            if (is_dyn(v)) return;
        const size_t a_size = r.n * r.c * r.hk * r.wk * r.hy * r.wy * ophip_dtype_nbytes(r.dt);
        if (ws && a_size <= max_ws) *ws = a_size;
    });
}

// Operator::launch (conv/im2col.rs:85-242)
int ophip_conv_launch(const ophip_conv *op, const ophip_conv_args *args, void *workspace, size_t workspace_len,
                      const ophip_queue_alloc *qa) {
    return guard([&] {
        if (!op || !args) throw args_not_support("null argument");
        const size_t hs = args->strides[0], ws = args->strides[1], hd = args->dilations[0], wd = args->dilations[1];
        no_padding(*args);
        const ConvMeta r = conv_meta(*args);
        const uint64_t dt = r.dt;
        const size_t n = static_of(r.n), m = static_of(r.m), c = static_of(r.c), h = static_of(r.h),
                     hy = static_of(r.hy), hk = static_of(r.hk), w = static_of(r.w), wy = static_of(r.wy),
                     wk = static_of(r.wk);
        const ptrdiff_t *ys = args->y_layout.strides, *xs = args->x_layout.strides, *ks = args->w_layout.strides;
        const ptrdiff_t nys = static_of(ys[0]), mys = static_of(ys[1]), hys = static_of(ys[2]), wys = static_of(ys[3]);
        const ptrdiff_t nxs = static_of(xs[0]), cxs = static_of(xs[1]), hxs = static_of(xs[2]), wxs = static_of(xs[3]);
        const ptrdiff_t mks = static_of(ks[0]), cks = static_of(ks[1]), hks = static_of(ks[2]), wks = static_of(ks[3]);
        const ptrdiff_t mbs = static_of(args->b_layout.strides[0]);
        if (hs == 0 || ws == 0 || hk == 0 || wk == 0) throw args_not_support("zero stride or kernel extent");

        // kernel extent with dilation
        const size_t hkd = (hk - 1) * hd + 1, wkd = (wk - 1) * wd + 1;
        if (h < hkd || w < wkd) throw shape_mismatch("kernel larger than the input");
        if ((h - hkd) % hs != 0 || (w - wkd) % ws != 0)
            throw strides_not_support("output size not divisible by strides");

        // c <- y: [n, m, hy * wy];  a <- w: [n, m, c * hk * wk];  b <- x: [n, c * hk * wk, hy * wy]
        size_t len;
        ptrdiff_t st;
        const size_t y_hw[2] = {hy, wy};
        const ptrdiff_t y_hw_s[2] = {hys, wys};
        if (!merge_be(y_hw, y_hw_s, 2, len, st)) throw strides_not_support("y rows and columns do not merge");
        const size_t cy_shape[3] = {n, m, hy * wy};
        const ptrdiff_t cy_strides[3] = {nys, mys, st};
        const size_t w_chw[3] = {c, hk, wk};
        const ptrdiff_t w_chw_s[3] = {cks, hks, wks};
        if (!merge_be(w_chw, w_chw_s, 3, len, st)) throw strides_not_support("w channels and taps do not merge");
        const size_t aw_shape[3] = {n, m, c * hk * wk};
        const ptrdiff_t aw_strides[3] = {0, mks, st};
        // x unfolded by a rearrange
        const ptrdiff_t ele = (ptrdiff_t)ophip_dtype_nbytes(dt);
        const size_t b_shape[6] = {n, c, hk, wk, hy, wy};
        const ptrdiff_t b_src_strides[6] = {nxs, cxs, hxs * (ptrdiff_t)hd, wxs * (ptrdiff_t)wd,
                                            hxs * (ptrdiff_t)hs, wxs * (ptrdiff_t)ws};
        ptrdiff_t b_dst_strides[6];
        ptrdiff_t mul = ele;
        for (int i = 6; i-- > 0;) {
            b_dst_strides[i] = mul;
            mul *= (ptrdiff_t)b_shape[i];
        }
        const size_t bx_shape[3] = {n, c * hk * wk, hy * wy};
        const ptrdiff_t bx_strides[3] = {b_dst_strides[0], b_dst_strides[3], ele};
        const ophip_tensor_layout c_y{dt, 3, cy_shape, cy_strides}, a_w{dt, 3, aw_shape, aw_strides},
            b_x{dt, 3, bx_shape, bx_strides}, b_dst{dt, 6, b_shape, b_dst_strides}, b_src{dt, 6, b_shape, b_src_strides};

        // the bias, broadcast over batch and positions
        const ptrdiff_t bias_strides[3] = {0, mbs, 0};
        const ophip_tensor_layout bias{dt, 3, cy_shape, bias_strides};
        const ophip_rearrange_args fill{c_y, args->y_base, bias, args->b_base};
        sub(ophip_rearrange_launch(op->rearrange, &fill, workspace, workspace_len, qa));

        // workspace for the unfolded x
        const size_t b_size = n * c * hk * wk * hy * wy * (size_t)ele;
        Workspace wsp(qa, workspace, workspace_len, b_size);
        char *b_mem = static_cast<char *>(wsp.ptr());
        const bool ext = wsp.ptr() == workspace && workspace_len >= b_size;
        void *rest = ext ? b_mem + b_size : nullptr;
        const size_t rest_len = ext ? workspace_len - b_size : 0;
        const ophip_rearrange_args unfold{b_dst, b_mem, b_src, args->x_base};
        sub(ophip_rearrange_launch(op->rearrange, &unfold, rest, rest_len, qa));

        const ophip_mat_mul_args mm{c_y, args->y_base, 1.f, a_w, args->w_base, b_x, b_mem, 1.f};
        sub(ophip_mat_mul_launch(op->mat_mul, &mm, rest, rest_len, qa));
    });
}

}  // extern "C"
