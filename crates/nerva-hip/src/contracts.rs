//! Names and properties of the rows this backend adds to the kernel-contract registry
//! (crates/nerva-kernel-contracts/src/registry/bootstrap.rs:39-108 holds the CUDA rows; the patch
//! beside this crate, kernel_contract_rows.patch, adds these). Kept here as plain data so that the
//! crate does not depend on the registry crate.

/// gfx target number the probe reports for the MI355X; the rows' architecture range is [950, 950].
pub const HIP_ARCH_GFX950: u32 = 950;

#[derive(Copy, Clone, Debug, Eq, PartialEq)]
pub struct HipContractRow {
    pub name: &'static str,
    pub operation: &'static str,
    pub dtypes: &'static [&'static str],
    pub graph_safe: bool,
    pub deterministic: bool,
    pub bit_exact: bool,
}

pub const HIP_CONTRACT_ROWS: &[HipContractRow] = &[
    HipContractRow {
        name: "hip_decode_dense_matvec_fp16_bf16",
        operation: "DenseMatVec",
        dtypes: &["F16", "BF16"],
        graph_safe: true,
        deterministic: true,
        bit_exact: false,
    },
    HipContractRow {
        name: "hip_decode_dense_matvec_fp8_e4m3",
        operation: "DenseMatVec",
        dtypes: &["F8E4M3"],
        graph_safe: true,
        deterministic: true,
        bit_exact: false,
    },
    HipContractRow {
        name: "hip_greedy_sample_u32",
        operation: "GreedySample",
        dtypes: &["U32"],
        graph_safe: true,
        deterministic: true,
        bit_exact: true,
    },
];
