//! Raw bindings to `libturbovec_hip.so`: one declaration per entry point of
//! `include/turbovec_hip.h`, same names, same argument order.
//!
//! Every function returns a `tv_status` as `c_int` (0 = ok); nothing unwinds across the
//! boundary.  Buffers are caller-owned host memory unless the name ends in `_dev`.  See the
//! header for what each entry point replaces in the turbovec crate (file:line), and
//! `rust/PATCH.md` for the call sites that change.
//!
//! Not compiled where this repository is built (no Rust toolchain there); kept equal to the
//! header by `tests/test_abi_host.py`.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_double, c_float, c_int, c_void};

/// Opaque device-resident index (codes, per-vector scales, rotation tables, centroids, TQ+ pair).
#[repr(C)]
pub struct tv_index {
    _private: [u8; 0],
}

// tv_status
pub const TV_OK: c_int = 0;
pub const TV_ERR_QUERY_BUFFER_NOT_MULTIPLE_OF_DIM: c_int = 1;
pub const TV_ERR_INVALID_QUERY_VALUE: c_int = 2;
pub const TV_ERR_MASK_LENGTH_MISMATCH: c_int = 3;
pub const TV_ERR_ALLOWLIST_EMPTY: c_int = 4;
pub const TV_ERR_UNKNOWN_ID: c_int = 5;
pub const TV_ERR_BAD_ARGUMENT: c_int = 6;
pub const TV_ERR_HIP: c_int = 7;
pub const TV_ERR_NO_DEVICE: c_int = 8;
pub const TV_ERR_INDEX_OUT_OF_RANGE: c_int = 9;
pub const TV_ERR_BAD_IMAGE: c_int = 10;

// tv_score_mode
pub const TV_SCORE_AUTO: c_int = 0;
pub const TV_SCORE_L_SCALAR: c_int = 1;
pub const TV_SCORE_L_CLASSIC: c_int = 2;
pub const TV_SCORE_L_U32: c_int = 3;
pub const TV_SCORE_P: c_int = 4;

extern "C" {
    pub fn tv_status_string(status: c_int) -> *const c_char;
    pub fn tv_last_error() -> *const c_char;

    // ---- index life cycle ----
    pub fn tv_index_create(dim: c_int, bits: c_int, device: c_int, out: *mut *mut tv_index) -> c_int;
    pub fn tv_index_destroy(ix: *mut tv_index) -> c_int;
    pub fn tv_index_set_tables(ix: *mut tv_index, signs: *const c_float, perms: *const u32, centroids: *const c_float) -> c_int;
    pub fn tv_index_set_calibration(ix: *mut tv_index, shift: *const c_float, scale: *const c_float) -> c_int;
    pub fn tv_index_set_score_mode(ix: *mut tv_index, mode: c_int) -> c_int;
    pub fn tv_index_get_tables(ix: *const tv_index, signs: *mut c_float, perms: *mut u32, centroids: *mut c_float, boundaries: *mut c_float) -> c_int;
    pub fn tv_index_upload_seq(ix: *mut tv_index, seq_codes: *const u8, n_vectors: usize, scales: *const c_float) -> c_int;
    pub fn tv_index_upload_seq_dev(ix: *mut tv_index, d_seq_codes: *const u8, n_vectors: usize, d_scales: *const c_float) -> c_int;
    pub fn tv_index_append_rows(ix: *mut tv_index, rows: *const u8, scales: *const c_float, n_new: usize) -> c_int;
    pub fn tv_index_add(ix: *mut tv_index, vectors: *const c_float, n_new: usize) -> c_int;
    pub fn tv_index_calibrate(ix: *mut tv_index, sample: *const c_float, n: usize) -> c_int;
    pub fn tv_index_get_calibration(ix: *const tv_index, shift: *mut c_float, scale: *mut c_float, n_calib: *mut usize) -> c_int;
    pub fn tv_index_add_dev(ix: *mut tv_index, d_vectors: *const c_float, n_new: usize) -> c_int;
    pub fn tv_index_swap_remove(ix: *mut tv_index, idx: usize) -> c_int;
    pub fn tv_index_download_seq(ix: *const tv_index, seq_out: *mut u8, scales_out: *mut c_float) -> c_int;
    pub fn tv_index_len(ix: *const tv_index) -> usize;
    pub fn tv_index_dim(ix: *const tv_index) -> c_int;
    pub fn tv_index_bits(ix: *const tv_index) -> c_int;

    // ---- search ----
    pub fn tv_validate_queries(queries: *const c_float, len: usize, dim: c_int, bad_index: *mut usize) -> c_int;
    pub fn tv_pack_mask(mask_bytes: *const u8, n: usize, words_out: *mut u64, n_allowed: *mut usize) -> c_int;
    pub fn tv_search(ix: *mut tv_index, queries: *const c_float, nq: usize, k: usize, mask_words: *const u64, n_mask_words: usize, out_scores: *mut c_float, out_indices: *mut i64, out_k_eff: *mut usize) -> c_int;
    pub fn tv_search_dev(ix: *mut tv_index, d_queries: *const c_float, nq: usize, k: usize, d_mask_words: *const u64, n_allowed: usize, d_out_scores: *mut c_float, d_out_indices: *mut i64, out_k_eff: *mut usize) -> c_int;
    pub fn tv_search_dev_noalloc(ix: *mut tv_index, d_queries: *const c_float, nq: usize, k: usize, d_mask_words: *const u64, n_allowed: usize, d_out_scores: *mut c_float, d_out_indices: *mut i64, out_k_eff: *mut usize) -> c_int;
    pub fn tv_noalloc_scratch_bytes() -> usize;

    // ---- host-only derivations ----
    pub fn tv_host_rotation_tables(dim: c_int, signs: *mut c_float, perms: *mut u32, block: *mut c_int, inv_sqrt_block: *mut c_float) -> c_int;
    pub fn tv_host_codebook(bits: c_int, dim: c_int, boundaries: *mut c_float, centroids: *mut c_float) -> c_int;

    // ---- snapshot images ----
    pub fn tv_host_snapshot_len(format: c_int, dim: c_int, bits: c_int, kind: c_int, n_calib: usize, n: usize) -> usize;
    pub fn tv_host_snapshot_compose(format: c_int, dim: c_int, bits: c_int, kind: c_int, boundaries: *const c_float, centroids: *const c_float, n_calib: usize, shift: *const c_float, scale: *const c_float, seq: *const u8, n: usize, scales: *const c_float, ids: *const u64, out: *mut u8) -> c_int;
    pub fn tv_host_snapshot_info(bytes: *const u8, len: usize, format: *mut c_int, kind: *mut c_int, dim: *mut c_int, bits: *mut c_int, n_calib: *mut usize, n: *mut usize) -> c_int;
    pub fn tv_host_snapshot_extract(bytes: *const u8, len: usize, boundaries: *mut c_float, centroids: *mut c_float, shift: *mut c_float, scale: *mut c_float, seq: *mut u8, scales: *mut c_float, ids: *mut u64) -> c_int;
    pub fn tv_index_to_bytes(ix: *const tv_index, ids: *const u64, format: c_int, out: *mut u8, cap: usize, len: *mut usize) -> c_int;
    pub fn tv_index_from_bytes(bytes: *const u8, len: usize, device: c_int, out: *mut *mut tv_index, ids_out: *mut u64) -> c_int;

    // ---- test / measurement hooks (not needed by a crate binding) ----
    pub fn tv_debug_scan(ix: *mut tv_index, queries: *const c_float, nq: usize, acc_out: *mut i32, scores_out: *mut c_float) -> c_int;
    pub fn tv_debug_prepare(ix: *mut tv_index, queries: *const c_float, nq: usize, q_rot_out: *mut c_float, scale_out: *mut c_float, bias_out: *mut c_float) -> c_int;
    pub fn tv_last_scan_ms(ix: *const tv_index, ms: *mut c_float, launches: *mut c_int) -> c_int;
    pub fn tv_debug_queries_per_launch(ix: *const tv_index, queries: *mut c_int) -> c_int;
    pub fn tv_debug_set_path(ix: *mut tv_index, force_full_lists: c_int) -> c_int;
    pub fn tv_debug_sampling_plan(ix: *const tv_index, nq: usize, k: usize, strides: *mut u32, repeat_offsets: *mut u32, cap: usize, count: *mut usize) -> c_int;
    pub fn tv_debug_level_repeats(ix: *mut tv_index, track: c_int, count: *mut usize) -> c_int;
    pub fn tv_debug_workspace_bytes(ix: *const tv_index, workspace: *mut usize, staging: *mut usize) -> c_int;
    pub fn tv_debug_overflow_redos(ix: *const tv_index, count: *mut usize) -> c_int;
    pub fn tv_debug_exact_redos(ix: *const tv_index, count: *mut usize) -> c_int;
    pub fn tv_debug_merged_calls(ix: *const tv_index, count: *mut usize) -> c_int;
    pub fn tv_debug_stream_probe(ix: *mut tv_index, d_src: *const c_void, d_dst: *mut c_void, bytes: usize, reps: c_int, ms_per_rep: *mut c_float) -> c_int;
    pub fn tv_debug_mfma_probe(ix: *mut tv_index, iters: c_int, reps: c_int, ms_per_rep: *mut c_float, ops_per_rep: *mut c_double) -> c_int;
    pub fn tv_index_device_ptrs(ix: *const tv_index, d_codes: *mut *mut c_void, d_scales: *mut *mut c_void, code_bytes: *mut usize) -> c_int;
}
