/*
 * CPU oracle for the quantized-matmul path -- TEST INFRASTRUCTURE ONLY
 * (tests, the smoke check and the benchmark's CPU-baseline leg).  See oracle.c.
 * Type codes equal the aclDataType values of include/acl/acl.h.
 */
#ifndef OPSNN_ORACLE_H_
#define OPSNN_ORACLE_H_
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

enum {
    ORC_F32 = 0, ORC_F16 = 1, ORC_I8 = 2, ORC_I32 = 3, ORC_BF16 = 27, ORC_I4 = 29,
    ORC_E5M2 = 35, ORC_E4M3 = 36, ORC_E8M0 = 37, ORC_E2M1 = 40, ORC_E1M2 = 41, ORC_U64 = 10
};

uint16_t orc_bf16_from_f32(float f);
float orc_bf16_to_f32(uint16_t h);
uint16_t orc_f16_from_f32(float f);
float orc_f16_to_f32(uint16_t h);
float orc_e4m3_to_f32(uint8_t b);
float orc_e5m2_to_f32(uint8_t b);
uint8_t orc_e4m3_from_f32(float f);
uint8_t orc_e5m2_from_f32(float f);
float orc_e2m1_to_f32(uint8_t code);
float orc_e8m0_to_f32(uint8_t b);
void orc_vec_f32_to_bf16(const float* in, uint16_t* out, size_t n);
void orc_vec_bf16_to_f32(const uint16_t* in, float* out, size_t n);
void orc_vec_f32_to_f16(const float* in, uint16_t* out, size_t n);
void orc_vec_f16_to_f32(const uint16_t* in, float* out, size_t n);
void orc_vec_f32_to_e4m3(const float* in, uint8_t* out, size_t n);
void orc_vec_e4m3_to_f32(const uint8_t* in, float* out, size_t n);
void orc_vec_e5m2_to_f32(const uint8_t* in, float* out, size_t n);
void orc_vec_e8m0_to_f32(const uint8_t* in, float* out, size_t n);
void orc_unpack_groupsize(int64_t gs, int64_t* gsM, int64_t* gsN, int64_t* gsK);
void orc_pack_int4_to_int32(const int8_t* in, int32_t* out, size_t n_packed);
void orc_unpack_int32_to_int4(const int32_t* in, int8_t* out, size_t n_packed);
void orc_convert_weight_b4(const int32_t* w, int64_t count, int is_fp32, uint8_t* out);
float orc_scale_generate(float s);
float orc_u64_to_deq_scale(uint64_t v);
size_t orc_dtype_bits(int dt);

int orc_qmm_int8_acc(const int8_t* x1, const int8_t* x2, int64_t M, int64_t K, int64_t N, int tA, int tB,
                     int32_t* acc);
int orc_qmm_pertoken_epilogue(const int32_t* acc, int64_t M, int64_t N, const float* x1s, const float* x2s,
                              int64_t x2s_len, const void* bias, int bias_dt, int y_dt, void* y);
int orc_qmm_pertoken(const int8_t* x1, const int8_t* x2, int64_t M, int64_t K, int64_t N, int tA, int tB,
                     const float* x1s, const float* x2s, int64_t x2s_len, const void* bias, int bias_dt, int y_dt,
                     void* y, int32_t* acc_out);
int orc_qmm_tc(const void* x1, const void* x2, int dt1, int dt2, int64_t M, int64_t K, int64_t N, int tA, int tB,
               const void* scale, int scale_dt, int64_t scale_len, const float* pertoken, const float* offset,
               int64_t offset_len, const void* bias, int bias_dt, int y_dt, void* y);
int orc_qmm_pertoken_f8(const void* x1, const void* x2, int dt1, int dt2, int64_t M, int64_t K, int64_t N, int tA, int tB,
                        const float* x1s, const float* x2s, int64_t x2s_len, const float* bias, int y_dt, void* y);
int orc_qmm_perblock(const void* x1, const void* x2, int dt1, int dt2, int64_t M, int64_t K, int64_t N, int tA,
                     int tB, const float* x1s, const float* x2s, int64_t gsM, int64_t gsN, int64_t gsK,
                     const float* bias, int y_dt, void* y);
int orc_qmm_mx(const void* x1, const void* x2, int dt1, int dt2, int64_t M, int64_t K, int64_t N, int tA, int tB,
               const uint8_t* x1s, const uint8_t* x2s, const float* bias, int y_dt, void* y);
int orc_qmm_tcg(const uint8_t* x1, const uint8_t* x2, int64_t M, int64_t K, int64_t N, int tB, const uint16_t* x2s,
                int s_dt, int64_t gs, const uint64_t* yscale, int64_t ylen, const float* bias, int y_dt, void* y);
int orc_qmm_i4_asym(const uint8_t* x1, const uint8_t* x2, int64_t M, int64_t K, int64_t N, int tB, const float* x1s,
                    const float* x2s, const uint16_t* x2o, int y_dt, void* y);
int orc_dynamic_quant(const void* x, int x_dt, int64_t rows, int64_t cols, const void* smooth, int y_dt, int symmetric,
                      void* y, float* scale_out, float* offset_out);
int orc_dynamic_quant_grouped(const void* x, int x_dt, int64_t rows, int64_t cols, const void* smooth, const int64_t* group_end,
                              int64_t groups, int y_dt, int symmetric, void* y, float* scale_out, float* offset_out);
int orc_dynamic_quant_wide(const void* x, int x_dt, int64_t rows, int64_t cols, int64_t chan_rows, int mode, const void* smooth, int y_dt,
                           int symmetric, void* y, float* scale_out, float* offset_out);
int orc_dynamic_block_quant(const void* x, int x_dt, int64_t batch, int64_t rows, int64_t cols, int64_t rb, int64_t cb,
                            double min_scale, int y_dt, uint8_t* y, float* scale_out);
int orc_dynamic_mx_quant(const void* x, int x_dt, int64_t rows, int64_t cols, int64_t block, int y_dt, uint8_t* y, uint8_t* scale_out);
void orc_trans_quant_param(const float* scale, int64_t scale_len, const float* offset, int64_t offset_len, int round_mode, uint64_t* out);
int orc_dynamic_mx_quant_alg(const void* x, int x_dt, int64_t rows, int64_t cols, int64_t block, int scale_alg, int y_dt, uint8_t* y,
                             uint8_t* scale_out);
int orc_dynamic_mx_quant_general(const void* x, int x_dt, int64_t outer, int64_t A, int64_t inner, int64_t block, int scale_alg,
                                 int round_mode, int y_dt, uint8_t* y, uint8_t* scale_out);
int orc_wqbmm(const void* x, int x_dt, const void* w, int w_dt, int64_t M, int64_t K, int64_t N, int tW,
              const void* scale, int scale_dt, int64_t scale_n, const void* offset, int64_t group,
              const void* bias, int bias_dt, void* y);

#ifdef __cplusplus
}
#endif
#endif
