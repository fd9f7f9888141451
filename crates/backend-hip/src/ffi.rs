//! Raw declarations of `include/eclat_hip.h`.  Source only: never compiled in this pipeline.
#![allow(non_camel_case_types)]

use std::ffi::{c_char, c_int, c_uint, c_void};

#[repr(C)] pub struct eh_device { _p: [u8; 0] }
#[repr(C)] pub struct eh_buffer { _p: [u8; 0] }
#[repr(C)] pub struct eh_program { _p: [u8; 0] }
#[repr(C)] pub struct eh_module { _p: [u8; 0] }
#[repr(C)] pub struct eh_plan { _p: [u8; 0] }

#[repr(C)]
pub struct eh_launch_info {
    pub entry: *const c_char,
    pub source: *const c_char,
    pub schedule: *const c_char,
    pub grid: [c_uint; 3],
    pub block: [c_uint; 3],
    pub lds_bytes: c_uint,
    pub n_args: c_int,
    pub n_kernels: c_int,
    pub algo_bytes: f64,
    pub flops: f64,
    pub lane: c_int,
    pub n_waits: c_int,
    pub tune_key: std::os::raw::c_ulonglong,
}

#[repr(C)]
pub struct eh_device_props {
    pub name: [c_char; 128],
    pub arch: [c_char; 32],
    pub compute_units: c_int,
    pub warp_size: c_int,
    pub max_work_group_size: c_int,
    pub local_memory_size: usize,
    pub global_memory_size: usize,
    pub clock_khz: c_int,
    pub memory_clock_khz: c_int,
    pub memory_bus_bits: c_int,
    pub l2_bytes: c_int,
}

unsafe extern "C" {
    pub fn eh_last_error() -> *const c_char;
    pub fn eh_free(p: *mut c_void);
    pub fn eh_render_program(ast_text: *const c_char, options: *const c_char, out: *mut *mut eh_plan) -> c_int;
    pub fn eh_plan_num_launches(plan: *mut eh_plan, n: *mut c_int) -> c_int;
    pub fn eh_plan_launch(plan: *mut eh_plan, launch: c_int, out: *mut eh_launch_info) -> c_int;
    pub fn eh_plan_release(plan: *mut eh_plan) -> c_int;
    pub fn eh_compile_source(source: *const c_char, arch: *const c_char, blob: *mut *mut c_void,
                             len: *mut usize) -> c_int;
    pub fn eh_device_count(count: *mut c_int) -> c_int;
    pub fn eh_device_open(index: c_int, out: *mut *mut eh_device) -> c_int;
    pub fn eh_device_close(dev: *mut eh_device) -> c_int;
    pub fn eh_device_get_props(dev: *mut eh_device, out: *mut eh_device_props) -> c_int;
    pub fn eh_buffer_alloc(dev: *mut eh_device, bytes: usize, out: *mut *mut eh_buffer) -> c_int;
    pub fn eh_buffer_release(buf: *mut eh_buffer) -> c_int;
    pub fn eh_buffer_write(buf: *mut eh_buffer, src: *const c_void, bytes: usize) -> c_int;
    pub fn eh_buffer_read(buf: *mut eh_buffer, dst: *mut c_void, bytes: usize) -> c_int;
    pub fn eh_buffer_copy(dst: *mut eh_buffer, src: *mut eh_buffer) -> c_int;
    pub fn eh_program_compile(dev: *mut eh_device, ast_text: *const c_char, options: *const c_char,
                              out: *mut *mut eh_program) -> c_int;
    pub fn eh_program_release(prog: *mut eh_program) -> c_int;
    pub fn eh_program_num_buffers(prog: *mut eh_program, n: *mut c_int) -> c_int;
    pub fn eh_program_buffer(prog: *mut eh_program, i: c_int, name: *mut *const c_char, role: *mut *const c_char,
                             bytes: *mut usize, elided: *mut c_int) -> c_int;
    pub fn eh_program_num_launches(prog: *mut eh_program, n: *mut c_int) -> c_int;
    pub fn eh_program_execute(prog: *mut eh_program, bufs: *const *mut eh_buffer, n_bufs: c_int, sync: c_int) -> c_int;
    pub fn eh_program_execute_positional(prog: *mut eh_program, inputs: *const *mut eh_buffer, n_in: c_int,
                                         outputs: *const *mut eh_buffer, n_out: c_int, sync: c_int) -> c_int;
    pub fn eh_program_binary(prog: *mut eh_program, launch: c_int, blob: *mut *const c_void,
                             len: *mut usize) -> c_int;
    pub fn eh_module_load(dev: *mut eh_device, blob: *const c_void, len: usize, entry: *const c_char,
                          out: *mut *mut eh_module) -> c_int;
    pub fn eh_module_launch(module: *mut eh_module, grid: *const c_uint, block: *const c_uint, lds_bytes: c_uint,
                            args: *const *mut eh_buffer, n_args: c_int, sync: c_int) -> c_int;
    pub fn eh_module_release(module: *mut eh_module) -> c_int;
}

pub fn last_error() -> String {
    unsafe {
        let p = eh_last_error();
        if p.is_null() { String::new() } else { std::ffi::CStr::from_ptr(p).to_string_lossy().into_owned() }
    }
}
