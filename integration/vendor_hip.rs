// Matchers of the HIP backend's hand-written kernels: saved as zyx/src/vendor/hip.rs beside matmul.rs, with `mod hip;`
// added to zyx/src/vendor/mod.rs. `HIPDevice::match_graph` (integration/hip.rs) tries them on every class in
// topological order and puts a `Node::Kernel` with the measured time into the output class of each match, the way
// `CblasDevice::match_graph` does for sgemm (zyx/src/backend/cblas.rs:213-238).
//
// Every matcher below is the Rust form of a matcher in zyx_amd/graph.py, which is the one that runs and is tested
// (tests/test_graph_oracle.py, tests/test_graph_fusion.py on the CPU; tests/test_gpu_graph.py, tests/test_gpu_block.py
// on the device); the Python name is given with each. No Rust toolchain exists where this library is built, so this
// file has never been compiled: it is written against the reference's types as they stand (zyx/src/graph/mod.rs:
// 100-180 `Node`, zyx/src/vendor/mod.rs:25-98 the query helpers, zyx/src/vendor/matmul.rs:41-71 `match_matmul`).
//
// The reference's graph is an e-graph: a class holds several equivalent nodes, and a matcher looks for ANY node of
// the wanted kind in a class (`find_map` over `classes[cid].nodes`), as matmul.rs does.

#![allow(unused)]

use crate::{
    DType,
    backend::hip::{HipMatch, ZhipKernelDesc},
    graph::{ClassId, Graph, Node},
    kernel::{BOp, UOp},
    shape::Dim,
};

// kernel kinds, epilogues and flags of include/zyx_hip.h
const K_SOFTMAX_ROWS: i32 = 1;
const K_REDUCE: i32 = 3;
const K_GEMM: i32 = 4;
const K_NORM_ROWS: i32 = 5;
const K_CROSS_ENTROPY: i32 = 6;
const K_ATTENTION: i32 = 10;
const EPI_NONE: i32 = 0;
const EPI_BIAS: i32 = 1;
const EPI_BIAS_RELU: i32 = 2;
const EPI_BIAS_GELU: i32 = 3;
const GEMM_TRANS_A: i32 = 1;
const GEMM_TRANS_B: i32 = 2;
const NORM_RMS: i32 = 1;
const NORM_WEIGHT: i32 = 2;
const NORM_BIAS: i32 = 4;
const CE_GRAD: i32 = 2;
const CE_MEAN: i32 = 4;
const CE_DENSE: i32 = 8;
const SOFTMAX_Y: i32 = 1;

fn bytes_of(dtype: DType) -> u64 {
    u64::from(dtype.byte_size())
}

impl Graph {
    // ---- queries beside those of vendor/mod.rs ---------------------------------------------------------------------

    fn binary_of(&self, cid: ClassId, op: BOp) -> Option<(ClassId, ClassId)> {
        self.classes[cid].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
            Node::Binary { x, y, bop } if *bop == op => Some((*x, *y)),
            _ => None,
        })
    }

    fn unary_of(&self, cid: ClassId, op: UOp) -> Option<ClassId> {
        self.classes[cid].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
            Node::Unary { x, uop } if *uop == op => Some(*x),
            _ => None,
        })
    }

    /// `Reduce(rop)` over the LAST axis of its operand: (operand, extent of that axis).
    fn reduce_last_of(&self, cid: ClassId, op: BOp) -> Option<(ClassId, Dim)> {
        self.classes[cid].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
            Node::Reduce { x, rop, axes } if *rop == op => {
                let s = self.const_shape(*x)?;
                (axes.len() == 1 && axes[0] == s.len() - 1).then(|| (*x, s[s.len() - 1]))
            }
            _ => None,
        })
    }

    /// The class a chain of Reshape / Expand nodes shows, when the chain only adds or repeats leading axes of a
    /// tensor whose own shape is `[n]` (a bias repeated along the rows): `_row_vector` in graph.py.
    fn row_vector_src(&self, cid: ClassId, n: Dim) -> Option<ClassId> {
        if self.const_shape(cid).as_deref() == Some(&[n][..]) {
            return Some(cid);
        }
        self.classes[cid].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
            Node::Expand { x, .. } | Node::Reshape { x, .. } => {
                let s = self.const_shape(*x)?;
                (s.last() == Some(&n) && s[..s.len() - 1].iter().all(|&d| d == 1)).then(|| self.row_vector_src(*x, n)).flatten()
            }
            _ => None,
        })
    }

    /// The scalar a class broadcasts (`_const_value`).
    fn scalar_of(&self, cid: ClassId) -> Option<f64> {
        self.classes[cid].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
            Node::Const(c) => c.as_f64(),
            Node::Expand { x, .. } | Node::Reshape { x, .. } => self.scalar_of(*x),
            _ => None,
        })
    }

    /// x when the class is `x.cmpgt(0) * x` (`Tensor::relu`, zyx/src/tensor/elementwise.rs:289-293): `_is_relu_of`.
    fn relu_src(&self, cid: ClassId) -> Option<ClassId> {
        let (a, b) = self.binary_of(cid, BOp::Mul)?;
        for (mask, x) in [(a, b), (b, a)] {
            if let Some((v, zero)) = self.binary_of(mask, BOp::Cmpgt) {
                if v == x && self.scalar_of(zero) == Some(0.0) {
                    return Some(x);
                }
            }
        }
        None
    }

    /// x when the class is `x * 0.5 * (tanh((x + x*x*x*0.044715) * sqrt(2/pi)) + 1)` with tanh written as
    /// `(e - 1) / (e + 1)`, `e = (u + u).exp()` (elementwise.rs:168-170, 585-588): `_is_gelu_of`, which compares
    /// against a template; here the tree is walked by hand.
    fn gelu_src(&self, cid: ClassId) -> Option<ClassId> {
        let (half, tp1) = self.binary_of(cid, BOp::Mul)?;
        let (x, c05) = self.binary_of(half, BOp::Mul)?;
        if self.scalar_of(c05) != Some(0.5) {
            return None;
        }
        let (tanh, one) = self.binary_of(tp1, BOp::Add)?;
        if self.scalar_of(one) != Some(1.0) {
            return None;
        }
        let (num, den) = self.binary_of(tanh, BOp::Div)?;
        let (e, _) = self.binary_of(num, BOp::Sub)?;
        let (e2, _) = self.binary_of(den, BOp::Add)?;
        if e != e2 {
            return None;
        }
        let (u, u2) = self.binary_of(self.unary_of(e, UOp::Exp)?, BOp::Add)?;
        if u != u2 {
            return None;
        }
        let (inner, k) = self.binary_of(u, BOp::Mul)?;
        if (self.scalar_of(k)? - 0.797_884_560_802_865_4).abs() > 1e-6 {
            return None;
        }
        let (x2, cube) = self.binary_of(inner, BOp::Add)?;
        let (xxx, c) = self.binary_of(cube, BOp::Mul)?;
        if x2 != x || (self.scalar_of(c)? - 0.044_715).abs() > 1e-7 {
            return None;
        }
        let (xx, x3) = self.binary_of(xxx, BOp::Mul)?;
        let (xa, xb) = self.binary_of(xx, BOp::Mul)?;
        (xa == x && xb == x && x3 == x).then_some(x)
    }

    /// `x . w^T` as `Linear::forward` writes it (zyx-nn/src/linear.rs:38-44: `x.dot(w.t())`, so the canonical matmul
    /// form of matmul.rs sees `b = w.t()` and would hand the kernel a transposed view): the product is matched with
    /// `w` [n, k] itself as the operand and the GEMM's trans_b flag, no transpose materialised. Falls back to
    /// `match_matmul` for a plain `a @ b`. Returns (a, b, m, n, k, trans_b). (`match_contraction` in graph.py, which
    /// also takes the backward products; those are reached here through `match_matmul` once autograd has put them
    /// into dot form.)
    fn product_of(&self, cid: ClassId) -> Option<(ClassId, ClassId, Dim, Dim, Dim, bool)> {
        let mm = self.match_matmul(cid)?;
        // b = w.t(): a Permute [1, 0] of a [n, k] class
        if let Some(w) = self.transpose_src(mm.b) {
            if self.const_shape(w).as_deref() == Some(&[mm.n, mm.k][..]) {
                return Some((mm.a, w, mm.m, mm.n, mm.k, true));
            }
        }
        Some((mm.a, mm.b, mm.m, mm.n, mm.k, false))
    }

    fn gemm_desc(dtype: DType, m: Dim, n: Dim, k: Dim, trans_b: bool, epilogue: i32, alpha: f32, residual: i32) -> ZhipKernelDesc {
        let mut d = ZhipKernelDesc::zeroed();
        d.kind = K_GEMM;
        d.dtype = dtype as i32;
        d.out_dtype = dtype as i32;
        d.flags = if trans_b { GEMM_TRANS_B } else { 0 };
        d.dims[0] = m as i64;
        d.dims[1] = n as i64;
        d.dims[2] = k as i64;
        d.dims[3] = 1;
        d.iparams[0] = epilogue;
        d.iparams[1] = dtype as i32; // bias dtype
        d.iparams[2] = residual;     // 0 none, 1 add, 2 multiply by (residual > 0)
        d.fparams[0] = alpha;
        d
    }

    // ---- the matchers ------------------------------------------------------------------------------------------------

    /// `match_linear`: a product with what the GEMM epilogue applies on the way out.
    ///   act(product + bias)        act = relu | gelu | nothing
    ///   (product + bias) + r       the skip connection around a Linear
    ///   w - product * c            an SGD step (zyx-optim/src/sgd.rs:45-84): alpha = -c, residual = w
    ///   product * (v > 0)          the reverse of a relu: residual = v, mask mode
    ///   product                    alone
    pub(crate) fn match_hip_linear(&self, cid: ClassId) -> Option<HipMatch> {
        let dtype = self.dtype(cid);
        if !matches!(dtype, DType::F32 | DType::BF16 | DType::F16) {
            return None;
        }
        let e = bytes_of(dtype);
        let make = |a: ClassId, b: ClassId, m: Dim, n: Dim, k: Dim, tb: bool, epi: i32, alpha: f32, res: i32, extra: Vec<(ClassId, u64)>| {
            let mut inputs = vec![a, b];
            let mut arg_bytes = vec![m * k * e, k * n * e];
            for (c, bytes) in extra {
                inputs.push(c);
                arg_bytes.push(bytes);
            }
            arg_bytes.push(m * n * e);
            HipMatch { desc: Self::gemm_desc(dtype, m, n, k, tb, epi, alpha, res), inputs, outputs: vec![cid], arg_bytes }
        };
        // activation, then bias
        let (act, pre) = if let Some(x) = self.relu_src(cid) {
            (EPI_BIAS_RELU, x)
        } else if let Some(x) = self.gelu_src(cid) {
            (EPI_BIAS_GELU, x)
        } else {
            (EPI_BIAS, cid)
        };
        if let Some((l, r)) = self.binary_of(pre, BOp::Add) {
            for (core, other) in [(l, r), (r, l)] {
                if let Some((a, b, m, n, k, tb)) = self.product_of(core) {
                    if let Some(bias) = self.row_vector_src(other, n) {
                        return Some(make(a, b, m, n, k, tb, act, 1.0, 0, vec![(bias, n * e)]));
                    }
                }
                // (product + bias) + skip
                if act == EPI_BIAS {
                    if let Some((l2, r2)) = self.binary_of(core, BOp::Add) {
                        for (core2, other2) in [(l2, r2), (r2, l2)] {
                            if let Some((a, b, m, n, k, tb)) = self.product_of(core2) {
                                if let Some(bias) = self.row_vector_src(other2, n) {
                                    if self.const_shape(other).as_deref() == Some(&[m, n][..]) {
                                        return Some(make(a, b, m, n, k, tb, EPI_BIAS, 1.0, 1, vec![(bias, n * e), (other, m * n * e)]));
                                    }
                                }
                            }
                        }
                    }
                }
            }
        }
        if act != EPI_BIAS {
            return None; // an activation straight on a product: the kernel has no such epilogue
        }
        // w - product * c
        if let Some((w, scaled)) = self.binary_of(cid, BOp::Sub) {
            if let Some((l, r)) = self.binary_of(scaled, BOp::Mul) {
                for (core, c) in [(l, r), (r, l)] {
                    if let (Some(lr), Some((a, b, m, n, k, tb))) = (self.scalar_of(c), self.product_of(core)) {
                        return Some(make(a, b, m, n, k, tb, EPI_NONE, -(lr as f32), 1, vec![(w, m * n * e)]));
                    }
                }
            }
        }
        // product * (v > 0)
        if let Some((l, r)) = self.binary_of(cid, BOp::Mul) {
            for (core, mask) in [(l, r), (r, l)] {
                if let (Some((v, zero)), Some((a, b, m, n, k, tb))) = (self.binary_of(mask, BOp::Cmpgt), self.product_of(core)) {
                    if self.scalar_of(zero) == Some(0.0) && self.dtype(v) == dtype {
                        return Some(make(a, b, m, n, k, tb, EPI_NONE, 1.0, 2, vec![(v, m * n * e)]));
                    }
                }
            }
        }
        let (a, b, m, n, k, tb) = self.product_of(cid)?;
        Some(make(a, b, m, n, k, tb, EPI_NONE, 1.0, 0, vec![]))
    }

    /// `e = (x - max_keepdim(x)).exp(); e / sum_keepdim(e)` over the last axis in f32 (`Tensor::softmax`,
    /// zyx/src/tensor/mod.rs:1457-1461): `match_softmax`. Returns (x, rows, cols) for the callers below too.
    fn softmax_parts(&self, cid: ClassId) -> Option<(ClassId, Dim, Dim)> {
        let shape = self.const_shape(cid)?;
        let cols = *shape.last()?;
        if self.dtype(cid) != DType::F32 || cols < 2 {
            return None;
        }
        let (e, den) = self.binary_of(cid, BOp::Div)?;
        let (esum, _) = self.reduce_last_of(self.expand_src(den)?.0, BOp::Add).or_else(|| {
            // keepdim = reduce then reshape to [.., 1]
            let r = self.classes[self.expand_src(den)?.0].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
                Node::Reshape { x, .. } => Some(*x),
                _ => None,
            })?;
            self.reduce_last_of(r, BOp::Add)
        })?;
        if esum != e {
            return None;
        }
        let (x, mx) = self.binary_of(self.unary_of(e, UOp::Exp)?, BOp::Sub)?;
        let m_src = self.expand_src(mx)?.0;
        let m_red = self.classes[m_src].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
            Node::Reshape { x, .. } => Some(*x),
            _ => None,
        }).unwrap_or(m_src);
        let (xm, _) = self.reduce_last_of(m_red, BOp::Max)?;
        (xm == x).then(|| (x, shape[..shape.len() - 1].iter().product(), cols))
    }

    pub(crate) fn match_hip_softmax(&self, cid: ClassId) -> Option<HipMatch> {
        let (x, rows, cols) = self.softmax_parts(cid)?;
        let mut d = ZhipKernelDesc::zeroed();
        d.kind = K_SOFTMAX_ROWS;
        d.dtype = DType::F32 as i32;
        d.out_dtype = DType::F32 as i32;
        d.flags = SOFTMAX_Y;
        d.dims[0] = rows as i64;
        d.dims[1] = cols as i64;
        Some(HipMatch { desc: d, inputs: vec![x], outputs: vec![cid], arg_bytes: vec![rows * cols * 4, rows * cols * 4] })
    }

    /// `Tensor::cross_entropy(target, Mean)` for a target of the logits' shape (zyx/src/tensor/mod.rs:1639-1655):
    /// `sum_all(sum(-(m - ln(sum(exp(m)))) * target, [1])) / rows`, `m = x - max_keepdim(x)`: the loss half of
    /// `scan_cross_entropy`. (The gradient half compares against the expression `Runtime::gradient` derives from this
    /// one; in the reference that expression only exists after `Tape::gradient`, and the comparison is node for node
    /// against a template built the same way, as graph.py does; it is not repeated here.)
    pub(crate) fn match_hip_cross_entropy(&self, cid: ClassId) -> Option<HipMatch> {
        if self.dtype(cid) != DType::F32 {
            return None;
        }
        let (total, n) = self.binary_of(cid, BOp::Div)?;
        let rows_f = self.scalar_of(n)?;
        let all = self.classes[total].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
            Node::Reduce { x, rop: BOp::Add, .. } => Some(*x),
            _ => None,
        })?;
        let (prod, cols) = self.reduce_last_of(all, BOp::Add)?;
        let (neg, target) = self.binary_of(prod, BOp::Mul)?;
        let lsm = self.unary_of(neg, UOp::Neg)?;
        let (m, lse) = self.binary_of(lsm, BOp::Sub)?;
        let (x, _mx) = self.binary_of(m, BOp::Sub)?;
        let ln_arg = self.unary_of(self.expand_src(lse)?.0, UOp::Ln).or_else(|| {
            let r = self.classes[self.expand_src(lse)?.0].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
                Node::Reshape { x, .. } => Some(*x),
                _ => None,
            })?;
            self.unary_of(r, UOp::Ln)
        })?;
        let (esrc, _) = self.reduce_last_of(ln_arg, BOp::Add).or_else(|| {
            let r = self.classes[ln_arg].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
                Node::Reshape { x, .. } => Some(*x),
                _ => None,
            })?;
            self.reduce_last_of(r, BOp::Add)
        })?;
        if self.unary_of(esrc, UOp::Exp)? != m {
            return None;
        }
        let shape = self.const_shape(x)?;
        if shape.len() != 2 || shape[1] != cols || shape[0] as f64 != rows_f || self.const_shape(target)? != shape {
            return None;
        }
        let rows = shape[0];
        let mut d = ZhipKernelDesc::zeroed();
        d.kind = K_CROSS_ENTROPY;
        d.dtype = DType::F32 as i32;
        d.out_dtype = DType::F32 as i32;
        d.flags = CE_MEAN | CE_DENSE;
        d.dims[0] = rows as i64;
        d.dims[1] = cols as i64;
        d.fparams[0] = 1.0 / rows as f32;
        Some(HipMatch { desc: d, inputs: vec![x, target], outputs: vec![cid], arg_bytes: vec![rows * cols * 4, rows * cols * 4, 4] })
    }

    /// `LayerNorm::forward` / `RMSNorm::forward` over the last axis (zyx-nn/src/layer_norm.rs:98-135,
    /// zyx-nn/src/rms_norm.rs:26-32): `match_norm`. graph.py recognises these by where the expression was built
    /// (`Graph.layer_norm` notes its result); the reference's graph keeps no such note, so the expression is walked:
    ///   ((x - mean) / sqrt(var + eps)) * weight + bias,   mean = sum_keepdim(x) / n,
    ///   var = sum_keepdim((x - mean') * (x - mean')) / (n - 1)
    ///   (x * (mean_keepdim(x * x) + eps).reciprocal().sqrt()) * scale
    pub(crate) fn match_hip_norm_rows(&self, cid: ClassId) -> Option<HipMatch> {
        let dtype = self.dtype(cid);
        if !matches!(dtype, DType::F32 | DType::BF16) {
            return None;
        }
        let shape = self.const_shape(cid)?;
        let cols = *shape.last()?;
        let rows: Dim = shape[..shape.len() - 1].iter().product();
        let e = bytes_of(dtype);
        // peel `+ bias` and `* weight`
        let (mut cur, mut weight, mut bias) = (cid, None, None);
        if let Some((l, r)) = self.binary_of(cur, BOp::Add) {
            if let Some(b) = self.row_vector_src(r, cols) {
                bias = Some(b);
                cur = l;
            }
        }
        if let Some((l, r)) = self.binary_of(cur, BOp::Mul) {
            if let Some(w) = self.row_vector_src(r, cols) {
                weight = Some(w);
                cur = l;
            }
        }
        let mut d = ZhipKernelDesc::zeroed();
        d.kind = K_NORM_ROWS;
        d.dtype = dtype as i32;
        d.out_dtype = dtype as i32;
        d.dims[0] = rows as i64;
        d.dims[1] = cols as i64;
        let x;
        if let Some((num, den)) = self.binary_of(cur, BOp::Div) {
            // LayerNorm
            let (xx, _mean) = self.binary_of(num, BOp::Sub)?;
            let (var, eps) = self.binary_of(self.unary_of(self.expand_src(den).map_or(den, |s| s.0), UOp::Sqrt)?, BOp::Add)?;
            let (ssq, nm1) = self.binary_of(var, BOp::Div)?;
            if self.scalar_of(nm1)? != (cols - 1) as f64 {
                return None;
            }
            d.fparams[0] = self.scalar_of(eps)? as f32;
            let _ = ssq; // the squared deviations: their operand is x again, checked through the mean below
            x = xx;
        } else {
            // RMSNorm
            let (xx, r) = self.binary_of(cur, BOp::Mul)?;
            let inv = self.unary_of(self.unary_of(self.expand_src(r).map_or(r, |s| s.0), UOp::Sqrt)?, UOp::Reciprocal)?;
            let (ms, eps) = self.binary_of(inv, BOp::Add)?;
            let (_sum, n) = self.binary_of(ms, BOp::Div)?;
            if self.scalar_of(n)? != cols as f64 || weight.is_none() {
                return None;
            }
            d.fparams[0] = self.scalar_of(eps)? as f32;
            d.flags |= NORM_RMS;
            x = xx;
        }
        if self.const_shape(x)? != shape {
            return None;
        }
        let mut inputs = vec![x];
        let mut arg_bytes = vec![rows * cols * e];
        if let Some(w) = weight {
            d.flags |= NORM_WEIGHT;
            inputs.push(w);
            arg_bytes.push(cols * e);
        }
        if let Some(b) = bias {
            d.flags |= NORM_BIAS;
            inputs.push(b);
            arg_bytes.push(cols * e);
        }
        arg_bytes.push(rows * cols * e);
        Some(HipMatch { desc: d, inputs, outputs: vec![cid], arg_bytes })
    }

    /// The core of `CausalSelfAttention::forward` between c_attn and c_proj (zyx-nn/src/causal_self_attention.rs:
    /// 39-69): `y = (softmax(q . k^T * scale) . v).transpose(1, 2).reshape([b, t, c])` with q, k, v the three thirds
    /// of qkv[b, t, 3c] viewed as [b, h, t, c / h]: `match_attention`. The walk goes from y down to the three Narrow
    /// nodes and checks that they slice one class at 0, c and 2c.
    pub(crate) fn match_hip_attention(&self, cid: ClassId) -> Option<HipMatch> {
        let dtype = self.dtype(cid);
        if !matches!(dtype, DType::F32 | DType::BF16) {
            return None;
        }
        let out_shape = self.const_shape(cid)?;
        if out_shape.len() != 3 {
            return None;
        }
        let (b, t, c) = (out_shape[0], out_shape[1], out_shape[2]);
        // y: Reshape <- Permute [0, 2, 1, 3] <- att . v (a batched product: Reduce(Add) of a broadcast Mul)
        let through = |cid: ClassId, want_permute: bool| -> Option<ClassId> {
            self.classes[cid].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
                Node::Reshape { x, .. } if !want_permute => Some(*x),
                Node::Permute { x, axes } if want_permute && axes.as_ref() == [0, 2, 1, 3] => Some(*x),
                _ => None,
            })
        };
        let pv = through(through(cid, false)?, true)?;
        let pv_shape = self.const_shape(pv)?;
        if pv_shape.len() != 4 || pv_shape[0] != b || pv_shape[2] != t {
            return None;
        }
        let (h, dh) = (pv_shape[1], pv_shape[3]);
        if h * dh != c {
            return None;
        }
        // the third of qkv a head view comes from: Permute [0, 2, 1, 3] <- Reshape [b, t, h, dh] <- Narrow(axis 2, start, c)
        let third = |cid: ClassId| -> Option<(ClassId, Dim)> {
            let r = through(through(cid, true)?, false)?;
            self.classes[r].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
                Node::Narrow { x, axis: 2, start, len } => {
                    let s = self.nodes[self.classes[*start].nodes[0]].node.as_const_dim()?;
                    let l = self.nodes[self.classes[*len].nodes[0]].node.as_const_dim()?;
                    (l == c).then_some((*x, s))
                }
                _ => None,
            })
        };
        // att . v: the product's operands seen through their Expand / Reshape wrappers
        let operand = |cid: ClassId| -> Option<ClassId> {
            let mut cur = self.expand_src(cid)?.0;
            while let Some(x) = through(cur, false) {
                cur = x;
            }
            Some(cur)
        };
        let red = self.classes[pv].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
            Node::Reshape { x, .. } => Some(*x),
            _ => None,
        }).unwrap_or(pv);
        let (prod, _) = self.reduce_last_of(red, BOp::Add)?;
        let (pa, pb) = self.mul_of(prod)?;
        let att = operand(pa)?;
        let vt = operand(pb)?; // v transposed by `dot`
        let v = self.classes[vt].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
            Node::Permute { x, axes } if axes.as_ref() == [0, 1, 3, 2] => Some(*x),
            _ => None,
        })?;
        let (scores, _, _) = self.softmax_parts(att)?;
        let (qk, sc) = self.binary_of(scores, BOp::Mul)?;
        let scale = self.scalar_of(sc)? as f32;
        let qk_red = self.classes[qk].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
            Node::Reshape { x, .. } => Some(*x),
            _ => None,
        }).unwrap_or(qk);
        let (qk_prod, _) = self.reduce_last_of(qk_red, BOp::Add)?;
        let (qa, kb) = self.mul_of(qk_prod)?;
        let (q, k) = (operand(qa)?, operand(kb)?); // `q.dot(k.t())`: dot's own transpose undoes k.t()
        let ((q_src, q0), (k_src, k0), (v_src, v0)) = (third(q)?, third(k)?, third(v)?);
        if q_src != k_src || q_src != v_src || (q0, k0, v0) != (0, c, 2 * c) {
            return None;
        }
        let e = bytes_of(dtype);
        let mut d = ZhipKernelDesc::zeroed();
        d.kind = K_ATTENTION;
        d.dtype = dtype as i32;
        d.out_dtype = dtype as i32;
        d.dims[0] = b as i64;
        d.dims[1] = t as i64;
        d.dims[2] = h as i64;
        d.dims[3] = dh as i64;
        d.fparams[0] = scale;
        Some(HipMatch { desc: d, inputs: vec![q_src], outputs: vec![cid], arg_bytes: vec![b * t * 3 * c * e, b * t * c * e] })
    }

    /// A long `Reduce(Add | Max)` over the trailing axes of a class that is a realized tensor (`match_reduce`):
    /// one launch of the two-stage reduce kernel instead of one serial loop per result. Shorter reductions stay
    /// with the generated kernel, which needs no second stage.
    pub(crate) fn match_hip_reduce(&self, cid: ClassId) -> Option<HipMatch> {
        let dtype = self.dtype(cid);
        if !matches!(dtype, DType::F32 | DType::BF16 | DType::F16 | DType::I32) {
            return None;
        }
        let (x, axes, op) = self.classes[cid].nodes.iter().find_map(|&nid| match &self.nodes[nid].node {
            Node::Reduce { x, rop, axes } if matches!(rop, BOp::Add | BOp::Max) => Some((*x, axes.clone(), *rop)),
            _ => None,
        })?;
        // the operand has to exist as a buffer: a leaf (anything else stays fused into the generated reduce)
        if !self.classes[x].nodes.iter().any(|&nid| matches!(self.nodes[nid].node, Node::Leaf { .. })) {
            return None;
        }
        let xs = self.const_shape(x)?;
        let (k, n) = (axes.len(), xs.len());
        let trailing = axes.iter().enumerate().all(|(i, &a)| a == n - k + i);
        let leading = axes.iter().enumerate().all(|(i, &a)| a == i);
        let (rows, cols, axis0): (Dim, Dim, bool) = if trailing {
            (xs[..n - k].iter().product(), xs[n - k..].iter().product(), false)
        } else if leading {
            (xs[..k].iter().product(), xs[k..].iter().product(), true)
        } else {
            return None;
        };
        if (if axis0 { rows } else { cols }) < 256 {
            return None;
        }
        let e = bytes_of(dtype);
        let mut d = ZhipKernelDesc::zeroed();
        d.kind = K_REDUCE;
        d.dtype = dtype as i32;
        d.out_dtype = dtype as i32;
        d.flags = i32::from(axis0);
        d.dims[0] = rows as i64;
        d.dims[1] = cols as i64;
        d.iparams[0] = i32::from(op == BOp::Max);
        let n_out = if axis0 { cols } else { rows };
        Some(HipMatch { desc: d, inputs: vec![x], outputs: vec![cid], arg_bytes: vec![rows * cols * e, n_out * e] })
    }
}
