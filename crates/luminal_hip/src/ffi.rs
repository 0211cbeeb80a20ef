//! `extern "C"` surface of libluminal_hip.so (include/luminal_hip.h), plus the status-to-panic bridge:
//! luminal's backends `unwrap()` every driver call, so a non-zero status becomes a panic here.
use std::ffi::{c_char, c_void, CStr};

pub type Status = i32;
pub type Stream = *mut c_void;

extern "C" {
    pub fn lhip_status_string(s: Status) -> *const c_char;
    pub fn lhip_last_hip_error() -> i32;
    pub fn lhip_init(device: i32) -> Status;
    pub fn lhip_malloc(dptr: *mut *mut c_void, nbytes: usize) -> Status;
    pub fn lhip_free(dptr: *mut c_void) -> Status;
    pub fn lhip_memcpy_h2d(dst: *mut c_void, src: *const c_void, nbytes: usize, s: Stream) -> Status;
    pub fn lhip_memcpy_d2h(dst: *mut c_void, src: *const c_void, nbytes: usize, s: Stream) -> Status;
    pub fn lhip_stream_sync(s: Stream) -> Status;
    pub fn lhip_q8_0_raw_nbytes(n: i64, k: i64) -> usize;
    pub fn lhip_q8_0_planar_nbytes(n: i64, k: i64) -> usize;
    pub fn lhip_q8_0_repack(raw: *const c_void, planar: *mut c_void, n: i64, k: i64, s: Stream) -> Status;
    // two planar (n, k) weights -> one planar (2n, k) weight, rows alternating: the (gate, up) order of the SwiGLU epilogue
    pub fn lhip_q8_0_interleave_rows(a: *const c_void, b: *const c_void, out: *mut c_void, n: i64, k: i64, s: Stream) -> Status;
    // batch-1 decode matvec with fusions: up to four weights on one activation row, optional RMS-norm prologue, epilogue
    // 0 none / 1 residual add / 2 SwiGLU over (gate, up) row pairs
    pub fn lhip_q8_0_matvec_fused_f32(w: *const *const c_void, y: *const *mut f32, n: *const i64, count: i32, x: *const f32, k: i64,
                                      norm_weight: *const f32, eps: f32, residual: *const f32, epilogue: i32, s: Stream) -> Status;
    // with more than a few rows (a prompt) both matmuls run on the matrix cores by themselves, at f32 accuracy, streaming the
    // weights once per 64 rows instead of once per row
    pub fn lhip_q8_0_matmul_f32(w: *const c_void, x: *const f32, y: *mut f32, m: i64, n: i64, k: i64, s: Stream) -> Status;
    pub fn lhip_q8_0_gather_f32(w: *const c_void, idx: *const f32, out: *mut f32, n_idx: i64, n: i64, k: i64, s: Stream) -> Status;
    // kernel-level route: names the kernel of luminal_hip_kernels.hsaco and the launch shape the matvec above would use, for a
    // host that drives hipModuleLoad / hipModuleGetFunction / hipModuleLaunchKernel itself (include/luminal_hip_kernels.h)
    pub fn lhip_q8_0_gemv_kernel_plan(n: i64, k: i64, f16: i32, kernel_name: *mut c_char, kernel_name_cap: usize,
                                      grid: *mut u32, block: *mut u32, lds_bytes: *mut u32) -> Status;
    // T = f16: x / y / out are IEEE binary16 buffers, sums stay f32
    pub fn lhip_q8_0_matmul_f16(w: *const c_void, x: *const c_void, y: *mut c_void, m: i64, n: i64, k: i64, s: Stream) -> Status;
    pub fn lhip_q8_0_gather_f16(w: *const c_void, idx: *const f32, out: *mut c_void, n_idx: i64, n: i64, k: i64, s: Stream) -> Status;
}

#[track_caller]
pub fn check(status: Status, what: &str) {
    if status != 0 {
        let name = unsafe { CStr::from_ptr(lhip_status_string(status)) }.to_string_lossy().into_owned();
        panic!("{what}: {name} (hipError_t {})", unsafe { lhip_last_hip_error() });
    }
}
