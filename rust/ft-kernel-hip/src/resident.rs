// Written by generate_bindings.py (static text). The device-resident surface, modelled on `ft_kernel_metal::fused`
// (crates/ft-kernel-metal/src/fused.rs:540-933, 986-1190): tensors live in HBM, every op enqueues on the batch's stream
// and returns a fresh resident tensor, `finish` is the only synchronisation.
use crate::ffi;

/// `ft_kernel_metal::Error` (crates/ft-kernel-metal/src/lib.rs:60-77) with the HIP backend's status codes behind it.
#[derive(Debug, Clone, PartialEq, Eq)]
pub enum Error {
    Unavailable,
    Kernel(String),
    SizeOverflow,
    BufferTooLarge,
    CommandBuffer(String),
}

fn check(rc: i32) -> Result<(), Error> {
    if rc == ffi::FTH_OK {
        return Ok(());
    }
    let mut info: ffi::fth_error_info = unsafe { std::mem::zeroed() };
    unsafe { ffi::fth_last_error(&mut info) };
    let end = info.message.iter().position(|&b| b == 0).unwrap_or(info.message.len());
    let text = String::from_utf8_lossy(&info.message[..end].iter().map(|&b| b as u8).collect::<Vec<u8>>()).into_owned();
    Err(match rc {
        ffi::FTH_ERR_UNAVAILABLE => Error::Unavailable,
        ffi::FTH_ERR_SIZE_OVERFLOW => Error::SizeOverflow,
        ffi::FTH_ERR_BUFFER_TOO_LARGE => Error::BufferTooLarge,
        ffi::FTH_ERR_STREAM => Error::CommandBuffer(text),
        _ => Error::Kernel(text),
    })
}

/// A resident f32 `[rows, cols]` matrix (`GpuTensor`, fused.rs:540-580): hipMalloc-backed, explicit copies.
pub struct HipTensor(*mut ffi::fth_tensor);
// The handle is only ever used through the library, which locks its own state (fused.rs:1018-1019 asserts the same).
unsafe impl Send for HipTensor {}
unsafe impl Sync for HipTensor {}

impl HipTensor {
    pub fn upload(host: &[f32], rows: usize, cols: usize) -> Result<Self, Error> {
        assert_eq!(host.len(), rows * cols);
        let mut t = std::ptr::null_mut();
        check(unsafe { ffi::fth_tensor_upload(host.as_ptr(), rows as i64, cols as i64, &mut t) })?;
        Ok(Self(t))
    }
    pub fn download(&self) -> Result<Vec<f32>, Error> {
        let (mut rows, mut cols) = (0i64, 0i64);
        check(unsafe { ffi::fth_tensor_shape(self.0, &mut rows, &mut cols) })?;
        let n = (rows * cols) as usize;
        let mut out = Vec::<f32>::with_capacity(n);
        check(unsafe { ffi::fth_tensor_download(self.0, out.as_mut_ptr(), n) })?;
        unsafe { out.set_len(n) };
        Ok(out)
    }
    pub(crate) fn raw(&self) -> *const ffi::fth_tensor {
        self.0
    }
}

impl Drop for HipTensor {
    fn drop(&mut self) {
        unsafe { ffi::fth_tensor_free(self.0) };
    }
}

/// A stream-ordered batch of ops (`Batch`, fused.rs:676-932).
pub struct Batch(*mut ffi::fth_batch);

impl Batch {
    pub fn new() -> Result<Self, Error> {
        let mut b = std::ptr::null_mut();
        check(unsafe { ffi::fth_batch_new(&mut b) })?;
        Ok(Self(b))
    }
    fn wrap(rc: i32, out: *mut ffi::fth_tensor) -> Result<HipTensor, Error> {
        check(rc).map(|()| HipTensor(out))
    }
    /// `y = a . w^T (+ bias)`, the weight in `nn.Linear`'s `[out, in]` layout (`Batch::matmul_bias`, fused.rs:676-762).
    pub fn linear(&mut self, a: &HipTensor, w: &HipTensor, bias: Option<&HipTensor>) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_linear(self.0, a.raw(), w.raw(), bias.map_or(std::ptr::null(), HipTensor::raw), &mut out) };
        Self::wrap(rc, out)
    }
    pub fn matmul(&mut self, a: &HipTensor, rhs: &HipTensor) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_matmul(self.0, a.raw(), rhs.raw(), &mut out) };
        Self::wrap(rc, out)
    }
    pub fn layernorm(&mut self, x: &HipTensor, gamma: &HipTensor, beta: &HipTensor, eps: f32) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_layernorm(self.0, x.raw(), gamma.raw(), beta.raw(), eps, &mut out) };
        Self::wrap(rc, out)
    }
    pub fn rmsnorm(&mut self, x: &HipTensor, gamma: &HipTensor, eps: f32) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_rmsnorm(self.0, x.raw(), gamma.raw(), eps, &mut out) };
        Self::wrap(rc, out)
    }
    pub fn gelu(&mut self, x: &HipTensor) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_gelu(self.0, x.raw(), &mut out) };
        Self::wrap(rc, out)
    }
    pub fn gelu_tanh(&mut self, x: &HipTensor) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_gelu_tanh(self.0, x.raw(), &mut out) };
        Self::wrap(rc, out)
    }
    pub fn add(&mut self, x: &HipTensor, y: &HipTensor) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_add(self.0, x.raw(), y.raw(), &mut out) };
        Self::wrap(rc, out)
    }
    pub fn softmax(&mut self, x: &HipTensor) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_softmax(self.0, x.raw(), &mut out) };
        Self::wrap(rc, out)
    }
    /// Multi-head attention over `[batch * seq, d_model]` q / k / v (`Batch::mha`, fused.rs:861-925).
    pub fn mha(&mut self, q: &HipTensor, k: &HipTensor, v: &HipTensor, n_heads: usize, batch: usize, causal: bool) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_mha(self.0, q.raw(), k.raw(), v.raw(), n_heads as i64, batch as i64, causal as i32, &mut out) };
        Self::wrap(rc, out)
    }
    /// The only synchronisation (`Batch::finish`, fused.rs:929-932).
    pub fn finish(&mut self) -> Result<(), Error> {
        check(unsafe { ffi::fth_batch_finish(self.0) })
    }
}

impl Drop for Batch {
    fn drop(&mut self) {
        unsafe { ffi::fth_batch_free(self.0) };
    }
}

/// One layer's weights as host slices, `nn.Linear` layout `[out, in]` (`LayerWeightsRef`, fused.rs:986-1016).
pub struct LayerWeightsRef<'a> {
    pub ln1_w: &'a [f32], pub ln1_b: &'a [f32],
    pub wq: &'a [f32], pub bq: &'a [f32], pub wk: &'a [f32], pub bk: &'a [f32], pub wv: &'a [f32], pub bv: &'a [f32],
    pub wo: &'a [f32], pub bo: &'a [f32],
    pub ln2_w: &'a [f32], pub ln2_b: &'a [f32],
    pub w1: &'a [f32], pub b1: &'a [f32], pub w2: &'a [f32], pub b2: &'a [f32],
}

/// Pre-LN encoder with resident weights (`EncoderGpu`, fused.rs:1024-1190).
pub struct EncoderHip {
    handle: *mut ffi::fth_encoder,
    d_model: usize,
}
unsafe impl Send for EncoderHip {}
unsafe impl Sync for EncoderHip {}

impl EncoderHip {
    pub fn new(d_model: usize, n_heads: usize, d_ff: usize, ln_eps: f32, causal: bool, layers: &[LayerWeightsRef<'_>]) -> Result<Self, Error> {
        let flat: Vec<ffi::fth_layer_weights> = layers
            .iter()
            .map(|l| ffi::fth_layer_weights {
                ln1_w: l.ln1_w.as_ptr(), ln1_b: l.ln1_b.as_ptr(),
                wq: l.wq.as_ptr(), bq: l.bq.as_ptr(), wk: l.wk.as_ptr(), bk: l.bk.as_ptr(), wv: l.wv.as_ptr(), bv: l.bv.as_ptr(),
                wo: l.wo.as_ptr(), bo: l.bo.as_ptr(),
                ln2_w: l.ln2_w.as_ptr(), ln2_b: l.ln2_b.as_ptr(),
                w1: l.w1.as_ptr(), b1: l.b1.as_ptr(), w2: l.w2.as_ptr(), b2: l.b2.as_ptr(),
            })
            .collect();
        let mut handle = std::ptr::null_mut();
        check(unsafe { ffi::fth_encoder_new(d_model as i64, n_heads as i64, d_ff as i64, ln_eps, causal as i32, flat.as_ptr(), flat.len() as i64, &mut handle) })?;
        Ok(Self { handle, d_model })
    }
    /// Host in, host out (`EncoderGpu::forward`, fused.rs:1136-1146).
    pub fn forward(&self, input: &[f32], batch: usize, seq: usize) -> Result<Vec<f32>, Error> {
        let n = batch * seq * self.d_model;
        assert_eq!(input.len(), n);
        let mut out = Vec::<f32>::with_capacity(n);
        check(unsafe { ffi::fth_encoder_forward(self.handle, input.as_ptr(), batch as i64, seq as i64, out.as_mut_ptr(), n) })?;
        unsafe { out.set_len(n) };
        Ok(out)
    }
}

impl Drop for EncoderHip {
    fn drop(&mut self) {
        unsafe { ffi::fth_encoder_free(self.handle) };
    }
}
