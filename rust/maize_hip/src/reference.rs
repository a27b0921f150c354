//! CPU twin of the product, for checking: C[i,j] = RNE_bf16( sum_k (f64)A[i,k] * (f64)B[k,j] ),
//! the mathematical intent of the reference mainloop (crates/maize_tile/src/gemm/mod.rs:37-90).
use crate::BF16;

/// One round-to-nearest-even from f64 to bf16 (NaN stays a quiet NaN, overflow goes to infinity).
pub fn bf16_from_f64(x: f64) -> BF16 {
    if x.is_nan() {
        return BF16(if x.is_sign_negative() { 0xFFC0 } else { 0x7FC0 });
    }
    // f64 -> f32 is itself a rounding, so round in f64 first: scale one bf16 quantum to 1.0.
    if x == 0.0 || x.is_infinite() {
        return BF16(((x as f32).to_bits() >> 16) as u16);
    }
    let e = ((x.abs().to_bits() >> 52) as i32 - 1023).max(-126); // floor(log2|x|), subnormal binade clamped
    let q = e - 7; // bf16 keeps 7 fraction bits
    let scaled = x * 2f64.powi(-q);
    let r = round_half_even(scaled);
    let v = (r * 2f64.powi(q)) as f32; // exact, or +-inf past the largest finite bf16
    BF16((v.to_bits() >> 16) as u16)
}

fn round_half_even(x: f64) -> f64 {
    let f = x.floor();
    let d = x - f;
    if d > 0.5 || (d == 0.5 && (f as i64) & 1 == 1) {
        f + 1.0
    } else {
        f
    }
}

/// Row-major A (m x k), B (k x n) -> C (m x n), fp64 accumulation in ascending k, one rounding.
pub fn gemm_nn(a: &[BF16], b: &[BF16], m: usize, n: usize, k: usize) -> Vec<BF16> {
    assert!(a.len() >= m * k && b.len() >= k * n);
    let bf: Vec<f64> = b.iter().map(|x| x.to_f32() as f64).collect();
    let mut c = vec![BF16(0); m * n];
    let mut acc = vec![0f64; n];
    for i in 0..m {
        acc.iter_mut().for_each(|x| *x = 0.0);
        for kk in 0..k {
            let av = a[i * k + kk].to_f32() as f64;
            let brow = &bf[kk * n..(kk + 1) * n];
            for (s, bv) in acc.iter_mut().zip(brow) {
                *s += av * bv; // bf16 x bf16 is exact in f64
            }
        }
        for j in 0..n {
            c[i * n + j] = bf16_from_f64(acc[j]);
        }
    }
    c
}

/// Distance in bf16 encodings (ordinal map: adjacent finite values differ by 1, +0 == -0).
pub fn ulp_distance(a: BF16, b: BF16) -> u32 {
    let ord = |h: u16| -> i32 {
        let mag = (h & 0x7FFF) as i32;
        if h & 0x8000 != 0 { -mag } else { mag }
    };
    (ord(a.0) - ord(b.0)).unsigned_abs()
}
