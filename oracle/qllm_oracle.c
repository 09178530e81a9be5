/*
 * CPU oracle for the speculative MTP-4 verify path.  TEST INFRASTRUCTURE ONLY:
 * loaded by tests/, by the smoke check and by the benchmark's cpu_baseline
 * leg; never linked into, or called from, the shipped HIP library.
 * See qllm_oracle.h for the reference file:line each function follows.
 */
#include "qllm_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

int qo_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---- scalar formats ---------------------------------------------------- */

static uint32_t f32_bits(float value) {
  uint32_t bits;
  memcpy(&bits, &value, sizeof bits);
  return bits;
}

static float bits_f32(uint32_t bits) {
  float value;
  memcpy(&value, &bits, sizeof value);
  return value;
}

float qo_bf16_round(float value) {
  uint32_t bits = f32_bits(value);
  if ((bits & 0x7f800000u) == 0x7f800000u) return value;
  bits += 0x7fffu + ((bits >> 16) & 1u);
  return bits_f32(bits & 0xffff0000u);
}

uint16_t qo_bf16_bits(float value) {
  uint32_t bits = f32_bits(value);
  if ((bits & 0x7f800000u) == 0x7f800000u) {
    /* keep NaN quiet and non-zero mantissa */
    uint16_t high = (uint16_t)(bits >> 16);
    if ((bits & 0x007fffffu) != 0u) high |= 0x0040u;
    return high;
  }
  bits += 0x7fffu + ((bits >> 16) & 1u);
  return (uint16_t)(bits >> 16);
}

float qo_bf16_value(uint16_t bits) { return bits_f32((uint32_t)bits << 16); }

uint16_t qo_f16_bits(float value) {
  const uint32_t bits = f32_bits(value);
  const uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
  const uint32_t magnitude = bits & 0x7fffffffu;
  if (magnitude >= 0x7f800000u) /* Inf / NaN */
    return (uint16_t)(sign | 0x7c00u |
                      (magnitude > 0x7f800000u ? 0x0200u : 0u));
  if (magnitude >= 0x477ff000u) /* rounds to >= 65520 -> Inf */
    return (uint16_t)(sign | 0x7c00u);
  if (magnitude < 0x33000001u) /* <= 2^-25: rounds to zero (tie to even) */
    return sign;
  const int exponent = (int)(magnitude >> 23) - 127;
  uint32_t mantissa = (magnitude & 0x007fffffu) | 0x00800000u;
  if (exponent < -14) {
    /* subnormal half: value = mantissa * 2^(exponent-23); unit 2^-24 */
    const int shift = -exponent - 1; /* 14..24 */
    const uint32_t kept = mantissa >> shift;
    const uint32_t rest = mantissa & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    uint32_t rounded = kept;
    if (rest > half || (rest == half && (kept & 1u))) ++rounded;
    return (uint16_t)(sign | rounded);
  }
  uint32_t kept = mantissa >> 13; /* 11 bits incl. hidden */
  const uint32_t rest = mantissa & 0x1fffu;
  if (rest > 0x1000u || (rest == 0x1000u && (kept & 1u))) ++kept;
  uint32_t half_exponent = (uint32_t)(exponent + 15);
  if (kept == 0x800u) { /* mantissa overflow */
    kept = 0x400u;
    ++half_exponent;
  }
  return (uint16_t)(sign | (half_exponent << 10) | (kept & 0x3ffu));
}

float qo_f16_value(uint16_t bits) {
  const uint32_t sign = ((uint32_t)bits & 0x8000u) << 16;
  const uint32_t exponent = (bits >> 10) & 0x1fu;
  const uint32_t mantissa = bits & 0x3ffu;
  if (exponent == 0x1fu)
    return bits_f32(sign | 0x7f800000u | (mantissa << 13));
  if (exponent == 0u) {
    const float magnitude = ldexpf((float)mantissa, -24);
    return sign ? -magnitude : magnitude;
  }
  return bits_f32(sign | ((exponent + 112u) << 23) | (mantissa << 13));
}

float qo_fp4_value(uint8_t code) {
  static const float levels[8] = {0.0f, 0.5f, 1.0f, 1.5f,
                                  2.0f, 3.0f, 4.0f, 6.0f};
  const float magnitude = levels[code & 7u];
  return (code & 8u) ? -magnitude : magnitude;
}

int qo_fp4_twice(uint8_t code) {
  static const int doubled[8] = {0, 1, 2, 3, 4, 6, 8, 12};
  const int magnitude = doubled[code & 7u];
  return (code & 8u) ? -magnitude : magnitude;
}

float qo_ue8m0_value(uint8_t code) {
  return code == 0u ? bits_f32(0x00400000u) : bits_f32((uint32_t)code << 23);
}

/* ---- FP4 matrices -------------------------------------------------------- */

static double block_scale(const void* scales, int scheme, uint32_t column) {
  if (scheme == QO_SCALE_F16_BLOCK16)
    return (double)qo_f16_value(((const uint16_t*)scales)[column / 16u]);
  return (double)qo_ue8m0_value(((const uint8_t*)scales)[column / 32u]);
}

static size_t scale_row_bytes(int scheme, uint32_t padded_columns) {
  return scheme == QO_SCALE_F16_BLOCK16 ? (size_t)(padded_columns / 16u) * 2u
                                        : (size_t)(padded_columns / 32u);
}

void qo_fp4_decode_row(const uint8_t* codes, const void* scales, int scheme,
                       uint32_t padded_columns, double* out) {
  for (uint32_t column = 0; column < padded_columns; ++column) {
    const uint8_t byte = codes[column / 2u];
    const uint8_t code = (column & 1u) ? (uint8_t)(byte >> 4) : (byte & 0x0fu);
    out[column] =
        (double)qo_fp4_value(code) * block_scale(scales, scheme, column);
  }
}

void qo_fp4_linear_f64(const uint8_t* codes, const void* scales, int scheme,
                       uint32_t rows, uint32_t padded_columns,
                       const float* act, uint32_t batch, float* out,
                       int bf16_output) {
  const size_t code_row = padded_columns / 2u;
  const size_t scale_row = scale_row_bytes(scheme, padded_columns);
#pragma omp parallel
  {
    double* weights = (double*)malloc(sizeof(double) * padded_columns);
#pragma omp for schedule(static)
    for (long row = 0; row < (long)rows; ++row) {
      qo_fp4_decode_row(codes + (size_t)row * code_row,
                        (const uint8_t*)scales + (size_t)row * scale_row,
                        scheme, padded_columns, weights);
      for (uint32_t request = 0; request < batch; ++request) {
        const float* x = act + (size_t)request * padded_columns;
        double sum = 0.0;
        for (uint32_t column = 0; column < padded_columns; ++column)
          sum += (double)x[column] * weights[column];
        float value = (float)sum;
        if (bf16_output) value = qo_bf16_round(value);
        out[(size_t)request * rows + (size_t)row] = value;
      }
    }
    free(weights);
  }
}

void qo_fp4_linear_block32_q8(const uint8_t* codes, const uint8_t* scales,
                              uint32_t rows, uint32_t padded_columns,
                              const int8_t* q8, const float* act_scales,
                              uint32_t batch, float* out, int bf16_output) {
  const uint32_t blocks = padded_columns / 32u;
#pragma omp parallel for schedule(static)
  for (long row = 0; row < (long)rows; ++row) {
    const uint8_t* row_codes = codes + (size_t)row * (padded_columns / 2u);
    const uint8_t* row_scales = scales + (size_t)row * blocks;
    for (uint32_t request = 0; request < batch; ++request) {
      const int8_t* x = q8 + (size_t)request * padded_columns;
      float total = 0.0f;
      for (uint32_t block = 0; block < blocks; ++block) {
        int32_t dot = 0;
        for (uint32_t index = 0; index < 32u; ++index) {
          const uint8_t byte = row_codes[block * 16u + index / 2u];
          const uint8_t code =
              (index & 1u) ? (uint8_t)(byte >> 4) : (byte & 0x0fu);
          dot += qo_fp4_twice(code) * (int32_t)x[block * 32u + index];
        }
        total += (float)dot * qo_ue8m0_value(row_scales[block]);
      }
      float value = total * act_scales[request] * 0.5f;
      if (bf16_output) value = qo_bf16_round(value);
      out[(size_t)request * rows + (size_t)row] = value;
    }
  }
}

void qo_quantize_q8_rows(const float* in, uint32_t rows, uint32_t columns,
                         uint32_t padded_columns, int bf16_input,
                         int8_t* out, float* scales) {
  for (uint32_t row = 0; row < rows; ++row) {
    const float* source = in + (size_t)row * columns;
    int8_t* target = out + (size_t)row * padded_columns;
    float maximum = 0.0f;
    for (uint32_t column = 0; column < columns; ++column) {
      const float value =
          bf16_input ? qo_bf16_round(source[column]) : source[column];
      maximum = fmaxf(maximum, fabsf(value));
    }
    const float scale = maximum > 0.0f ? maximum / 127.0f : 1.0f;
    scales[row] = scale;
    for (uint32_t column = 0; column < padded_columns; ++column) {
      int quantized = 0;
      if (column < columns) {
        const float value =
            bf16_input ? qo_bf16_round(source[column]) : source[column];
        quantized = (int)nearbyintf(value / scale);
      }
      if (quantized > 127) quantized = 127;
      if (quantized < -127) quantized = -127;
      target[column] = (int8_t)quantized;
    }
  }
}

void qo_fp4_embedding(const uint8_t* codes, const void* scales, int scheme,
                      uint32_t columns, uint32_t padded_columns,
                      const uint32_t* tokens, uint32_t batch, float* out) {
  const size_t code_row = padded_columns / 2u;
  const size_t scale_row = scale_row_bytes(scheme, padded_columns);
  double* weights = (double*)malloc(sizeof(double) * padded_columns);
  for (uint32_t request = 0; request < batch; ++request) {
    const size_t token = tokens[request];
    qo_fp4_decode_row(codes + token * code_row,
                      (const uint8_t*)scales + token * scale_row, scheme,
                      padded_columns, weights);
    for (uint32_t column = 0; column < columns; ++column)
      out[(size_t)request * columns + column] = (float)weights[column];
  }
  free(weights);
}

/* ---- normalisation and elementwise ------------------------------------- */

void qo_rms_norm_rows(const float* in, const float* weight, float* out,
                      uint32_t rows, uint32_t elements, float epsilon,
                      int zero_centered, int bf16_output) {
  for (uint32_t row = 0; row < rows; ++row) {
    const float* x = in + (size_t)row * elements;
    float* y = out + (size_t)row * elements;
    double square = 0.0;
    for (uint32_t index = 0; index < elements; ++index)
      square += (double)x[index] * (double)x[index];
    const double inverse =
        1.0 / sqrt(square / (double)elements + (double)epsilon);
    for (uint32_t index = 0; index < elements; ++index) {
      double factor = 1.0;
      if (weight)
        factor = zero_centered ? 1.0 + (double)weight[index]
                               : (double)weight[index];
      float value = (float)((double)x[index] * inverse * factor);
      y[index] = bf16_output ? qo_bf16_round(value) : value;
    }
  }
}

void qo_silu_product(const float* gate, const float* up, float* out,
                     uint32_t elements, int bf16_activations) {
  for (uint32_t index = 0; index < elements; ++index) {
    const double g = (double)gate[index];
    float activated = (float)(g / (1.0 + exp(-g)));
    if (bf16_activations) activated = qo_bf16_round(activated);
    float value = (float)((double)activated * (double)up[index]);
    out[index] = bf16_activations ? qo_bf16_round(value) : value;
  }
}

void qo_add_in_place(float* destination, const float* source,
                     uint32_t elements, int bf16_output) {
  for (uint32_t index = 0; index < elements; ++index) {
    const float value = destination[index] + source[index];
    destination[index] = bf16_output ? qo_bf16_round(value) : value;
  }
}

/* ---- attention preparation ---------------------------------------------- */

void qo_head_norm_rope(float* x, const float* weight, uint32_t head_dim,
                       uint32_t rotary_dim, uint32_t position, float epsilon,
                       float theta, int bf16_activations) {
  double* normalized = (double*)malloc(sizeof(double) * head_dim);
  if (weight) {
    double square = 0.0;
    for (uint32_t index = 0; index < head_dim; ++index)
      square += (double)x[index] * (double)x[index];
    const double inverse =
        1.0 / sqrt(square / (double)head_dim + (double)epsilon);
    for (uint32_t index = 0; index < head_dim; ++index) {
      float value =
          (float)((double)x[index] * inverse * (1.0 + (double)weight[index]));
      normalized[index] =
          bf16_activations ? (double)qo_bf16_round(value) : (double)value;
    }
  } else {
    for (uint32_t index = 0; index < head_dim; ++index)
      normalized[index] = (double)x[index];
  }
  const uint32_t half = rotary_dim / 2u;
  for (uint32_t index = 0; index < head_dim; ++index) {
    double result = normalized[index];
    if (index < rotary_dim) {
      const uint32_t pair = index % half;
      const double angle =
          (double)position *
          pow((double)theta, -2.0 * (double)pair / (double)rotary_dim);
      const double other =
          index < half ? -normalized[index + half] : normalized[index - half];
      double cosine = cos(angle);
      double sine = sin(angle);
      if (bf16_activations) {
        cosine = (double)qo_bf16_round((float)cosine);
        sine = (double)qo_bf16_round((float)sine);
      }
      result = normalized[index] * cosine + other * sine;
    }
    const float value = (float)result;
    x[index] = bf16_activations ? qo_bf16_round(value) : value;
  }
  free(normalized);
}

size_t qo_q4h_layer_bytes(uint32_t page_tokens, uint32_t kv_heads,
                          uint32_t head_dim) {
  return (size_t)page_tokens * kv_heads * 2u * (head_dim / 2u + 2u);
}

struct q4h_planes {
  uint8_t* key_codes;
  uint8_t* key_scales;
  uint8_t* value_codes;
  uint8_t* value_scales;
};

static struct q4h_planes q4h_planes_of(uint8_t* page, uint32_t layer,
                                       uint32_t page_tokens,
                                       uint32_t kv_heads,
                                       uint32_t head_dim) {
  const size_t records = (size_t)page_tokens * kv_heads;
  struct q4h_planes planes;
  planes.key_codes =
      page + (size_t)layer * qo_q4h_layer_bytes(page_tokens, kv_heads, head_dim);
  planes.key_scales = planes.key_codes + records * (head_dim / 2u);
  planes.value_codes = planes.key_scales + records * 2u;
  planes.value_scales = planes.value_codes + records * (head_dim / 2u);
  return planes;
}

static void q4h_encode(const float* x, uint32_t head_dim, uint8_t* codes,
                       uint8_t* scale_bytes) {
  float maximum = 0.0f;
  for (uint32_t index = 0; index < head_dim; ++index)
    maximum = fmaxf(maximum, fabsf(x[index]));
  const uint16_t bits = qo_f16_bits(fmaxf(maximum / 7.0f, 0x1p-24f));
  const float scale = qo_f16_value(bits);
  memcpy(scale_bytes, &bits, 2);
  for (uint32_t index = 0; index < head_dim; index += 2u) {
    int low = (int)nearbyintf(x[index] / scale);
    int high = (int)nearbyintf(x[index + 1u] / scale);
    low = low < -7 ? -7 : (low > 7 ? 7 : low);
    high = high < -7 ? -7 : (high > 7 ? 7 : high);
    codes[index / 2u] = (uint8_t)((low & 0x0f) | ((high & 0x0f) << 4));
  }
}

void qo_q4h_store(uint8_t* page, uint32_t layer, uint32_t page_tokens,
                  uint32_t cache_position, uint32_t kv_head,
                  uint32_t kv_heads, uint32_t head_dim, const float* key,
                  const float* value) {
  const struct q4h_planes planes =
      q4h_planes_of(page, layer, page_tokens, kv_heads, head_dim);
  const size_t record =
      (size_t)kv_head * page_tokens + cache_position % page_tokens;
  q4h_encode(key, head_dim, planes.key_codes + record * (head_dim / 2u),
             planes.key_scales + record * 2u);
  q4h_encode(value, head_dim, planes.value_codes + record * (head_dim / 2u),
             planes.value_scales + record * 2u);
}

static int signed_nibble(uint8_t nibble) {
  return nibble >= 8u ? (int)nibble - 16 : (int)nibble;
}

static void q4h_codes_of(const uint8_t* codes, uint32_t head_dim, int* out) {
  for (uint32_t index = 0; index < head_dim; ++index) {
    const uint8_t byte = codes[index / 2u];
    out[index] = signed_nibble((index & 1u) ? (uint8_t)(byte >> 4)
                                            : (uint8_t)(byte & 0x0fu));
  }
}

void qo_q4h_load(const uint8_t* page, uint32_t layer, uint32_t page_tokens,
                 uint32_t cache_position, uint32_t kv_head,
                 uint32_t kv_heads, uint32_t head_dim, float* key,
                 float* value) {
  const struct q4h_planes planes = q4h_planes_of(
      (uint8_t*)(uintptr_t)page, layer, page_tokens, kv_heads, head_dim);
  const size_t record =
      (size_t)kv_head * page_tokens + cache_position % page_tokens;
  uint16_t key_bits, value_bits;
  memcpy(&key_bits, planes.key_scales + record * 2u, 2);
  memcpy(&value_bits, planes.value_scales + record * 2u, 2);
  const float key_scale = qo_f16_value(key_bits);
  const float value_scale = qo_f16_value(value_bits);
  int* codes = (int*)malloc(sizeof(int) * head_dim);
  q4h_codes_of(planes.key_codes + record * (head_dim / 2u), head_dim, codes);
  for (uint32_t index = 0; index < head_dim; ++index)
    key[index] = (float)codes[index] * key_scale;
  q4h_codes_of(planes.value_codes + record * (head_dim / 2u), head_dim, codes);
  for (uint32_t index = 0; index < head_dim; ++index)
    value[index] = (float)codes[index] * value_scale;
  free(codes);
}

void qo_quantize_queries_q8(const float* queries, uint32_t rows,
                            uint32_t query_heads, uint32_t head_dim,
                            uint32_t query_stride, int8_t* q8,
                            float* scales) {
  for (uint32_t row = 0; row < rows; ++row) {
    for (uint32_t head = 0; head < query_heads; ++head) {
      const size_t record = (size_t)row * query_heads + head;
      const float* source = queries + record * query_stride;
      float maximum = 0.0f;
      for (uint32_t index = 0; index < head_dim; ++index)
        maximum = fmaxf(maximum, fabsf(source[index]));
      const float scale = fmaxf(maximum / 127.0f, 0x1p-24f);
      scales[record] = scale;
      for (uint32_t index = 0; index < head_dim; ++index) {
        int quantized = (int)nearbyintf(source[index] / scale);
        quantized = quantized < -127 ? -127 : (quantized > 127 ? 127 : quantized);
        q8[record * head_dim + index] = (int8_t)quantized;
      }
    }
  }
}

/* ---- attention ------------------------------------------------------------ */

static uint32_t query_stride_of(const struct qo_attention_shape* shape) {
  return (shape->output_gated ? 2u : 1u) * shape->head_dim;
}

void qo_attention_q4h_f64(const struct qo_attention_shape* shape,
                          const float* queries,
                          const uint8_t* const* page_table, float* out) {
  const uint32_t d = shape->head_dim;
  const uint32_t group = shape->query_heads / shape->kv_heads;
  const uint32_t stride = query_stride_of(shape);
  const uint32_t last_context = shape->first_context_tokens + shape->rows - 1u;
#pragma omp parallel for schedule(dynamic, 1)
  for (long kv_head = 0; kv_head < (long)shape->kv_heads; ++kv_head) {
    float* keys = (float*)malloc(sizeof(float) * (size_t)last_context * d);
    float* values = (float*)malloc(sizeof(float) * (size_t)last_context * d);
    for (uint32_t token = 0; token < last_context; ++token)
      qo_q4h_load(page_table[token / shape->page_tokens], shape->layer,
                  shape->page_tokens, token, (uint32_t)kv_head,
                  shape->kv_heads, d, keys + (size_t)token * d,
                  values + (size_t)token * d);
    double* scores = (double*)malloc(sizeof(double) * last_context);
    double* accumulator = (double*)malloc(sizeof(double) * d);
    for (uint32_t row = 0; row < shape->rows; ++row) {
      const uint32_t context = shape->first_context_tokens + row;
      for (uint32_t local = 0; local < group; ++local) {
        const uint32_t head = (uint32_t)kv_head * group + local;
        const size_t record = (size_t)row * shape->query_heads + head;
        const float* q = queries + record * stride;
        double maximum = -INFINITY;
        for (uint32_t token = 0; token < context; ++token) {
          const float* k = keys + (size_t)token * d;
          double dot = 0.0;
          for (uint32_t index = 0; index < d; ++index)
            dot += (double)q[index] * (double)k[index];
          scores[token] = dot / sqrt((double)d);
          if (scores[token] > maximum) maximum = scores[token];
        }
        double denominator = 0.0;
        for (uint32_t index = 0; index < d; ++index) accumulator[index] = 0.0;
        for (uint32_t token = 0; token < context; ++token) {
          const double p = exp(scores[token] - maximum);
          denominator += p;
          const float* v = values + (size_t)token * d;
          for (uint32_t index = 0; index < d; ++index)
            accumulator[index] += p * (double)v[index];
        }
        for (uint32_t index = 0; index < d; ++index) {
          double result = accumulator[index] / denominator;
          if (shape->output_gated)
            result /= 1.0 + exp(-(double)q[d + index]);
          out[record * d + index] = (float)result;
        }
      }
    }
    free(scores);
    free(accumulator);
    free(keys);
    free(values);
  }
}

void qo_attention_q4h_int8(const struct qo_attention_shape* shape,
                           const float* queries,
                           const uint8_t* const* page_table, float* out) {
  const uint32_t d = shape->head_dim;
  const uint32_t group = shape->query_heads / shape->kv_heads;
  const uint32_t stride = query_stride_of(shape);
  const size_t query_records = (size_t)shape->rows * shape->query_heads;
  int8_t* q8 = (int8_t*)malloc(query_records * d);
  float* q_scales = (float*)malloc(sizeof(float) * query_records);
  qo_quantize_queries_q8(queries, shape->rows, shape->query_heads, d, stride,
                         q8, q_scales);
  const float score_scale = 1.0f / sqrtf((float)d);
  const uint32_t last_context = shape->first_context_tokens + shape->rows - 1u;
  float* scores = (float*)malloc(sizeof(float) * last_context);
  float* probabilities = (float*)malloc(sizeof(float) * last_context);
  float* value_scales = (float*)malloc(sizeof(float) * last_context);
  int* quantized = (int*)malloc(sizeof(int) * last_context);
  int* codes = (int*)malloc(sizeof(int) * d);
  int* value_codes = (int*)malloc(sizeof(int) * (size_t)last_context * d);
  for (uint32_t row = 0; row < shape->rows; ++row) {
    const uint32_t context = shape->first_context_tokens + row;
    for (uint32_t head = 0; head < shape->query_heads; ++head) {
      const uint32_t kv_head = head / group;
      const size_t record = (size_t)row * shape->query_heads + head;
      float maximum = -INFINITY;
      for (uint32_t token = 0; token < context; ++token) {
        const uint8_t* page = page_table[token / shape->page_tokens];
        const struct q4h_planes planes =
            q4h_planes_of((uint8_t*)(uintptr_t)page, shape->layer,
                          shape->page_tokens, shape->kv_heads, d);
        const size_t plane_record =
            (size_t)kv_head * shape->page_tokens + token % shape->page_tokens;
        uint16_t key_bits, value_bits;
        memcpy(&key_bits, planes.key_scales + plane_record * 2u, 2);
        memcpy(&value_bits, planes.value_scales + plane_record * 2u, 2);
        q4h_codes_of(planes.key_codes + plane_record * (d / 2u), d, codes);
        int32_t dot = 0;
        for (uint32_t index = 0; index < d; ++index)
          dot += (int32_t)q8[record * d + index] * codes[index];
        scores[token] = ((float)dot * q_scales[record] *
                         qo_f16_value(key_bits)) * score_scale;
        maximum = fmaxf(maximum, scores[token]);
        value_scales[token] = qo_f16_value(value_bits);
        q4h_codes_of(planes.value_codes + plane_record * (d / 2u), d,
                     value_codes + (size_t)token * d);
      }
      float denominator = 0.0f;
      float weighted_maximum = 0.0f;
      for (uint32_t token = 0; token < context; ++token) {
        probabilities[token] = expf(scores[token] - maximum);
        denominator += probabilities[token];
        weighted_maximum =
            fmaxf(weighted_maximum, probabilities[token] * value_scales[token]);
      }
      const float probability_scale =
          fmaxf(weighted_maximum / 127.0f, 0x1p-24f);
      for (uint32_t token = 0; token < context; ++token) {
        int q = (int)nearbyintf(probabilities[token] * value_scales[token] /
                                probability_scale);
        quantized[token] = q < 0 ? 0 : (q > 127 ? 127 : q);
      }
      for (uint32_t index = 0; index < d; ++index) {
        int32_t product = 0;
        for (uint32_t token = 0; token < context; ++token)
          product += quantized[token] * value_codes[(size_t)token * d + index];
        float result = ((float)product * probability_scale) / denominator;
        if (shape->output_gated)
          result /= 1.0f + expf(-queries[record * stride + d + index]);
        out[record * d + index] = result;
      }
    }
  }
  free(value_codes);
  free(codes);
  free(quantized);
  free(value_scales);
  free(probabilities);
  free(scores);
  free(q_scales);
  free(q8);
}

size_t qo_q8_layer_bytes(uint32_t page_tokens, uint32_t kv_heads,
                         uint32_t head_dim) {
  return (size_t)2u * page_tokens * kv_heads * (head_dim + 2u);
}

static void q8_encode(uint8_t* record, const float* x, uint32_t d) {
  float maximum = 0.0f;
  for (uint32_t index = 0; index < d; ++index) {
    const float magnitude = fabsf(x[index]);
    if (magnitude > maximum) maximum = magnitude;
  }
  const uint16_t scale_bits = qo_f16_bits(fmaxf(maximum / 127.0f, 0x1p-24f));
  const float scale = qo_f16_value(scale_bits);
  for (uint32_t index = 0; index < d; ++index) {
    int code = (int)nearbyintf(x[index] / scale);
    if (code > 127) code = 127;
    if (code < -127) code = -127;
    record[index] = (uint8_t)(int8_t)code;
  }
  memcpy(record + d, &scale_bits, sizeof(scale_bits));
}

static void q8_decode(const uint8_t* record, uint32_t d, float* x) {
  uint16_t scale_bits;
  memcpy(&scale_bits, record + d, sizeof(scale_bits));
  const float scale = qo_f16_value(scale_bits);
  for (uint32_t index = 0; index < d; ++index)
    x[index] = (float)(int8_t)record[index] * scale;
}

void qo_q8_store(uint8_t* page, size_t layer_offset, uint32_t page_tokens,
                 uint32_t position, uint32_t kv_head, uint32_t kv_heads,
                 uint32_t head_dim, const float* key, const float* value) {
  const size_t record_bytes = head_dim + 2u;
  const size_t records = (size_t)page_tokens * kv_heads;
  const size_t record = (size_t)(position % page_tokens) * kv_heads + kv_head;
  uint8_t* keys = page + layer_offset;
  q8_encode(keys + record * record_bytes, key, head_dim);
  q8_encode(keys + (records + record) * record_bytes, value, head_dim);
}

void qo_q8_load(const uint8_t* page, size_t layer_offset, uint32_t page_tokens,
                uint32_t position, uint32_t kv_head, uint32_t kv_heads,
                uint32_t head_dim, float* key, float* value) {
  const size_t record_bytes = head_dim + 2u;
  const size_t records = (size_t)page_tokens * kv_heads;
  const size_t record = (size_t)(position % page_tokens) * kv_heads + kv_head;
  const uint8_t* keys = page + layer_offset;
  q8_decode(keys + record * record_bytes, head_dim, key);
  q8_decode(keys + (records + record) * record_bytes, head_dim, value);
}

void qo_attention_q8_f64(const struct qo_attention_shape* shape,
                         size_t layer_offset, const float* queries,
                         const uint8_t* const* page_table, float* out) {
  const uint32_t d = shape->head_dim;
  const uint32_t group = shape->query_heads / shape->kv_heads;
  const uint32_t stride = query_stride_of(shape);
  const uint32_t last_context = shape->first_context_tokens + shape->rows - 1u;
#pragma omp parallel for schedule(dynamic, 1)
  for (long kv_index = 0; kv_index < (long)shape->kv_heads; ++kv_index) {
    const uint32_t kv_head = (uint32_t)kv_index;
    float* keys = (float*)malloc(sizeof(float) * (size_t)last_context * d);
    float* values = (float*)malloc(sizeof(float) * (size_t)last_context * d);
    double* scores = (double*)malloc(sizeof(double) * last_context);
    double* accumulator = (double*)malloc(sizeof(double) * d);
    for (uint32_t token = 0; token < last_context; ++token)
      qo_q8_load(page_table[token / shape->page_tokens], layer_offset,
                 shape->page_tokens, token, kv_head, shape->kv_heads, d,
                 keys + (size_t)token * d, values + (size_t)token * d);
    for (uint32_t member = 0; member < group; ++member) {
      const uint32_t head = kv_head * group + member;
      for (uint32_t row = 0; row < shape->rows; ++row) {
        const uint32_t context = shape->first_context_tokens + row;
        const size_t record = (size_t)row * shape->query_heads + head;
        const float* q = queries + record * stride;
        double maximum = -INFINITY;
        for (uint32_t token = 0; token < context; ++token) {
          double dot = 0.0;
          for (uint32_t index = 0; index < d; ++index)
            dot += (double)q[index] * (double)keys[(size_t)token * d + index];
          scores[token] = dot / sqrt((double)d);
          if (scores[token] > maximum) maximum = scores[token];
        }
        double denominator = 0.0;
        for (uint32_t index = 0; index < d; ++index) accumulator[index] = 0.0;
        for (uint32_t token = 0; token < context; ++token) {
          const double p = exp(scores[token] - maximum);
          denominator += p;
          for (uint32_t index = 0; index < d; ++index)
            accumulator[index] += p * (double)values[(size_t)token * d + index];
        }
        for (uint32_t index = 0; index < d; ++index) {
          double result = accumulator[index] / denominator;
          if (shape->output_gated)
            result /= 1.0 + exp(-(double)q[d + index]);
          out[record * d + index] = (float)result;
        }
      }
    }
    free(keys);
    free(values);
    free(scores);
    free(accumulator);
  }
}

void qo_attention_f16_f64(const struct qo_attention_shape* shape,
                          const float* queries,
                          const uint8_t* const* page_table,
                          int f16_probabilities, float* out) {
  const uint32_t d = shape->head_dim;
  const uint32_t group = shape->query_heads / shape->kv_heads;
  const uint32_t stride = query_stride_of(shape);
  const size_t page_values = (size_t)shape->page_tokens * shape->kv_heads * d;
  const uint32_t last_context = shape->first_context_tokens + shape->rows - 1u;
#pragma omp parallel for schedule(dynamic, 1)
  for (long head_index = 0; head_index < (long)shape->query_heads;
       ++head_index) {
    const uint32_t head = (uint32_t)head_index;
    const uint32_t kv_head = head / group;
    double* scores = (double*)malloc(sizeof(double) * last_context);
    double* accumulator = (double*)malloc(sizeof(double) * d);
    for (uint32_t row = 0; row < shape->rows; ++row) {
      const uint32_t context = shape->first_context_tokens + row;
      const size_t record = (size_t)row * shape->query_heads + head;
      const float* q = queries + record * stride;
      double maximum = -INFINITY;
      for (uint32_t token = 0; token < context; ++token) {
        const uint16_t* layer_keys =
            (const uint16_t*)page_table[token / shape->page_tokens] +
            (size_t)shape->layer * 2u * page_values;
        const uint16_t* k =
            layer_keys +
            ((size_t)(token % shape->page_tokens) * shape->kv_heads + kv_head) *
                d;
        double dot = 0.0;
        for (uint32_t index = 0; index < d; ++index) {
          const float query =
              f16_probabilities ? qo_f16_value(qo_f16_bits(q[index])) : q[index];
          dot += (double)query * (double)qo_f16_value(k[index]);
        }
        if (f16_probabilities)
          scores[token] = (double)((float)dot * (1.0f / sqrtf((float)d)));
        else
          scores[token] = dot / sqrt((double)d);
        if (scores[token] > maximum) maximum = scores[token];
      }
      double denominator = 0.0;
      for (uint32_t index = 0; index < d; ++index) accumulator[index] = 0.0;
      for (uint32_t token = 0; token < context; ++token) {
        double p = exp(scores[token] - maximum);
        if (f16_probabilities)
          p = (double)qo_f16_value(qo_f16_bits((float)p));
        denominator += p;
        const uint16_t* layer_values =
            (const uint16_t*)page_table[token / shape->page_tokens] +
            (size_t)shape->layer * 2u * page_values + page_values;
        const uint16_t* v =
            layer_values +
            ((size_t)(token % shape->page_tokens) * shape->kv_heads + kv_head) *
                d;
        for (uint32_t index = 0; index < d; ++index)
          accumulator[index] += p * (double)qo_f16_value(v[index]);
      }
      for (uint32_t index = 0; index < d; ++index) {
        double result = accumulator[index] / denominator;
        if (shape->output_gated)
          result /= 1.0 + exp(-(double)q[d + index]);
        out[record * d + index] = (float)result;
      }
    }
    free(scores);
    free(accumulator);
  }
}

void qo_attention_combine(const float* partial_maxima,
                          const float* partial_sums,
                          const float* partial_outputs, const float* gate,
                          uint32_t gate_stride, uint32_t rows,
                          uint32_t query_heads, uint32_t head_dim,
                          uint32_t first_context_tokens,
                          uint32_t split_tokens, uint32_t maximum_splits,
                          float* out) {
  for (uint32_t row = 0; row < rows; ++row) {
    const uint32_t active =
        (first_context_tokens + row + split_tokens - 1u) / split_tokens;
    for (uint32_t head = 0; head < query_heads; ++head) {
      float maximum = -INFINITY;
      for (uint32_t split = 0; split < active; ++split)
        maximum = fmaxf(
            maximum,
            partial_maxima[((size_t)row * maximum_splits + split) * query_heads +
                           head]);
      float sum = 0.0f;
      for (uint32_t split = 0; split < active; ++split) {
        const size_t partial =
            ((size_t)row * maximum_splits + split) * query_heads + head;
        sum += partial_sums[partial] * expf(partial_maxima[partial] - maximum);
      }
      for (uint32_t index = 0; index < head_dim; ++index) {
        float result = 0.0f;
        for (uint32_t split = 0; split < active; ++split) {
          const size_t partial =
              ((size_t)row * maximum_splits + split) * query_heads + head;
          result += partial_outputs[partial * head_dim + index] *
                    expf(partial_maxima[partial] - maximum);
        }
        result /= sum;
        const size_t record = (size_t)row * query_heads + head;
        if (gate)
          result *= 1.0f / (1.0f + expf(-gate[record * gate_stride + index]));
        out[record * head_dim + index] = result;
      }
    }
  }
}

/* ---- token selection ------------------------------------------------------- */

uint32_t qo_argmax(const float* values, uint32_t count) {
  float best = -INFINITY;
  uint32_t index = 0xffffffffu;
  for (uint32_t item = 0; item < count; ++item) {
    const float value = values[item];
    if (value > best || (value == best && item < index)) {
      best = value;
      index = item;
    }
  }
  return index;
}

uint32_t qo_topk(const float* values, uint32_t count, uint32_t k,
                 float* out_values, uint32_t* out_indices) {
  /* k sequential exact selections, each excluding earlier winners. */
  uint8_t* taken = (uint8_t*)calloc(count, 1);
  uint32_t written = 0;
  for (uint32_t rank = 0; rank < k; ++rank) {
    float best = -INFINITY;
    uint32_t index = 0xffffffffu;
    for (uint32_t item = 0; item < count; ++item) {
      const float value = values[item];
      if (taken[item] || isnan(value)) continue;
      if (value > best || (value == best && item < index)) {
        best = value;
        index = item;
      }
    }
    if (index == 0xffffffffu) break;
    taken[index] = 1;
    out_values[written] = best;
    out_indices[written] = index;
    ++written;
  }
  free(taken);
  return written;
}

void qo_presence_penalty(float* logits, const uint8_t* emitted,
                         uint32_t count, float penalty) {
  for (uint32_t index = 0; index < count; ++index)
    if (emitted[index] != 0u) logits[index] -= penalty;
}

/* ---- sampling ---------------------------------------------------------------- */

static int compare_u32(const void* a, const void* b) {
  const uint32_t x = *(const uint32_t*)a;
  const uint32_t y = *(const uint32_t*)b;
  return x < y ? -1 : (x > y ? 1 : 0);
}

static int validate_distribution(const struct qo_token_probability* entries,
                                 uint32_t count) {
  if (count == 0u) return QO_INVALID_ARGUMENT;
  double total = 0.0;
  uint32_t* tokens = (uint32_t*)malloc(sizeof(uint32_t) * count);
  for (uint32_t index = 0; index < count; ++index) {
    const double p = entries[index].probability;
    if (!isfinite(p) || p < 0.0) {
      free(tokens);
      return QO_INVALID_ARGUMENT;
    }
    total += p;
    tokens[index] = entries[index].token;
  }
  qsort(tokens, count, sizeof(uint32_t), compare_u32);
  int duplicate = 0;
  for (uint32_t index = 1; index < count; ++index)
    if (tokens[index] == tokens[index - 1u]) duplicate = 1;
  free(tokens);
  if (duplicate || !isfinite(total) || fabs(total - 1.0) > 1e-10)
    return QO_INVALID_ARGUMENT;
  return QO_OK;
}

static double probability_of(const struct qo_token_probability* entries,
                             uint32_t count, uint32_t token) {
  for (uint32_t index = 0; index < count; ++index)
    if (entries[index].token == token) return entries[index].probability;
  return 0.0;
}

int qo_make_sampling_distribution(const float* sorted_logits,
                                  const uint32_t* sorted_tokens,
                                  uint32_t count, uint32_t temperature_ppm,
                                  uint32_t top_p_ppm, uint32_t min_p_ppm,
                                  struct qo_token_probability* entries,
                                  uint32_t* out_count) {
  if (count == 0u || temperature_ppm == 0u || temperature_ppm > 2000000u ||
      top_p_ppm == 0u || top_p_ppm > 1000000u || min_p_ppm > 1000000u ||
      !isfinite(sorted_logits[0]))
    return QO_INVALID_ARGUMENT;
  for (uint32_t index = 1; index < count; ++index) {
    const float previous = sorted_logits[index - 1u];
    const float current = sorted_logits[index];
    if ((!isnan(current) && current > previous) ||
        (current == previous && sorted_tokens[index] < sorted_tokens[index - 1u]))
      return QO_INVALID_ARGUMENT;
  }
  const double inverse_temperature = 1000000.0 / (double)temperature_ppm;
  const double maximum = (double)sorted_logits[0];
  const double minimum_relative = (double)min_p_ppm / 1000000.0;
  double* weights = (double*)malloc(sizeof(double) * count);
  uint32_t kept = 0;
  double total = 0.0;
  for (uint32_t index = 0; index < count; ++index) {
    const double logit = (double)sorted_logits[index];
    const double weight =
        isfinite(logit) ? exp((logit - maximum) * inverse_temperature) : 0.0;
    if (weight < minimum_relative) continue;
    entries[kept].token = sorted_tokens[index];
    weights[kept] = weight;
    total += weight;
    ++kept;
  }
  if (kept == 0u || !isfinite(total) || !(total > 0.0)) {
    free(weights);
    return QO_INVALID_ARGUMENT;
  }
  const double top_p = (double)top_p_ppm / 1000000.0;
  double cumulative = 0.0;
  uint32_t nucleus = kept;
  for (uint32_t index = 0; index < kept; ++index) {
    cumulative += weights[index] / total;
    if (cumulative >= top_p) {
      nucleus = index + 1u;
      break;
    }
  }
  total = 0.0;
  for (uint32_t index = 0; index < nucleus; ++index) total += weights[index];
  for (uint32_t index = 0; index < nucleus; ++index)
    entries[index].probability = weights[index] / total;
  *out_count = nucleus;
  free(weights);
  return QO_OK;
}

static int uniform_ok(double value) {
  return isfinite(value) && value >= 0.0 && value < 1.0;
}

int qo_sample_distribution(const struct qo_token_probability* entries,
                           uint32_t count, double uniform,
                           uint32_t* out_token) {
  int status = validate_distribution(entries, count);
  if (status != QO_OK) return status;
  if (!uniform_ok(uniform)) return QO_INVALID_ARGUMENT;
  double cumulative = 0.0;
  for (uint32_t index = 0; index < count; ++index) {
    cumulative += entries[index].probability;
    if (uniform < cumulative) {
      *out_token = entries[index].token;
      return QO_OK;
    }
  }
  *out_token = entries[count - 1u].token;
  return QO_OK;
}

struct residual_entry {
  uint32_t token;
  uint32_t order; /* insertion order, for a stable sort by token */
  double target;
  double draft;
  int has_draft;
};

static int compare_residual(const void* a, const void* b) {
  const struct residual_entry* x = (const struct residual_entry*)a;
  const struct residual_entry* y = (const struct residual_entry*)b;
  if (x->token != y->token) return x->token < y->token ? -1 : 1;
  return x->order < y->order ? -1 : (x->order > y->order ? 1 : 0);
}

int qo_rejection_sample(uint32_t proposal,
                        const struct qo_token_probability* target,
                        uint32_t target_count,
                        const struct qo_token_probability* draft,
                        uint32_t draft_count, double acceptance_uniform,
                        double correction_uniform,
                        struct qo_rejection_result* result) {
  int status = validate_distribution(target, target_count);
  if (status != QO_OK) return status;
  status = validate_distribution(draft, draft_count);
  if (status != QO_OK) return status;
  if (!uniform_ok(acceptance_uniform) || !uniform_ok(correction_uniform))
    return QO_INVALID_ARGUMENT;
  const double target_probability =
      probability_of(target, target_count, proposal);
  const double draft_probability = probability_of(draft, draft_count, proposal);
  if (!(draft_probability > 0.0)) return QO_INVALID_ARGUMENT;
  double acceptance = target_probability / draft_probability;
  if (acceptance > 1.0) acceptance = 1.0;
  result->target_probability = target_probability;
  result->draft_probability = draft_probability;
  if (acceptance_uniform < acceptance) {
    result->accepted = 1;
    result->token = proposal;
    return QO_OK;
  }
  /* residual[token] = target; then for each draft entry
   * residual[token] = max(0, residual[token] - q); walked in ascending id. */
  const uint32_t total_entries = target_count + draft_count;
  struct residual_entry* merged =
      (struct residual_entry*)malloc(sizeof(*merged) * total_entries);
  for (uint32_t index = 0; index < target_count; ++index) {
    merged[index].token = target[index].token;
    merged[index].order = index;
    merged[index].target = target[index].probability;
    merged[index].draft = 0.0;
    merged[index].has_draft = 0;
  }
  for (uint32_t index = 0; index < draft_count; ++index) {
    struct residual_entry* entry = &merged[target_count + index];
    entry->token = draft[index].token;
    entry->order = target_count + index;
    entry->target = 0.0;
    entry->draft = draft[index].probability;
    entry->has_draft = 1;
  }
  qsort(merged, total_entries, sizeof(*merged), compare_residual);
  /* collapse equal tokens (a target entry sorts before its draft entry) */
  uint32_t unique = 0;
  for (uint32_t index = 0; index < total_entries;) {
    double value = 0.0;
    uint32_t next = index;
    const uint32_t token = merged[index].token;
    while (next < total_entries && merged[next].token == token) {
      if (merged[next].has_draft)
        value = fmax(0.0, value - merged[next].draft);
      else
        value = merged[next].target;
      ++next;
    }
    merged[unique].token = token;
    merged[unique].target = value;
    ++unique;
    index = next;
  }
  double total = 0.0;
  for (uint32_t index = 0; index < unique; ++index)
    total += merged[index].target;
  if (!isfinite(total) || !(total > 0.0)) {
    free(merged);
    return QO_RUNTIME_ERROR;
  }
  const double threshold = correction_uniform * total;
  double cumulative = 0.0;
  uint32_t last_positive = 0;
  int found_positive = 0;
  for (uint32_t index = 0; index < unique; ++index) {
    if (merged[index].target > 0.0) {
      last_positive = merged[index].token;
      found_positive = 1;
    }
    cumulative += merged[index].target;
    if (threshold < cumulative) {
      result->accepted = 0;
      result->token = merged[index].token;
      free(merged);
      return QO_OK;
    }
  }
  free(merged);
  if (!found_positive) return QO_RUNTIME_ERROR;
  result->accepted = 0;
  result->token = last_positive;
  return QO_OK;
}

static uint64_t splitmix64(uint64_t value) {
  value += 0x9e3779b97f4a7c15ull;
  value = (value ^ (value >> 30)) * 0xbf58476d1ce4e5b9ull;
  value = (value ^ (value >> 27)) * 0x94d049bb133111ebull;
  return value ^ (value >> 31);
}

double qo_counter_uniform(uint64_t seed, uint32_t position, uint32_t stream,
                          uint32_t index) {
  uint64_t counter = seed;
  counter ^= (uint64_t)position * 0xd2b74407b1ce6e93ull;
  counter ^= (uint64_t)stream * 0xca5a826395121157ull;
  counter ^= (uint64_t)index * 0x9e3779b185ebca87ull;
  return (double)(splitmix64(counter) >> 11) * (1.0 / 9007199254740992.0);
}

/* ---- acceptance ------------------------------------------------------------------ */

struct qo_verify_result qo_accept_greedy(const float* logits,
                                         uint32_t vocabulary,
                                         const uint32_t* drafts,
                                         uint32_t draft_count) {
  struct qo_verify_result result = {0u, 0u, QO_OK};
  for (uint32_t row = 0; row < draft_count; ++row) {
    const uint32_t best = qo_argmax(logits + (size_t)row * vocabulary, vocabulary);
    if (best != drafts[row]) {
      result.accepted = row;
      result.next_token = best;
      return result;
    }
  }
  result.accepted = draft_count;
  result.next_token =
      qo_argmax(logits + (size_t)draft_count * vocabulary, vocabulary);
  return result;
}

struct qo_verify_result qo_accept_stochastic(
    const struct qo_token_probability* const* target,
    const uint32_t* target_counts,
    const struct qo_token_probability* const* draft,
    const uint32_t* draft_counts, const uint32_t* drafts,
    uint32_t draft_count, uint64_t seed, uint32_t position) {
  struct qo_verify_result result = {0u, 0u, QO_OK};
  uint32_t accepted = 0;
  for (; accepted < draft_count; ++accepted) {
    struct qo_rejection_result decision;
    const int status = qo_rejection_sample(
        drafts[accepted], target[accepted], target_counts[accepted],
        draft[accepted], draft_counts[accepted],
        qo_counter_uniform(seed, position + accepted, 100u, accepted),
        qo_counter_uniform(seed, position + accepted, 200u, accepted),
        &decision);
    if (status != QO_OK) {
      result.status = status;
      result.accepted = accepted;
      return result;
    }
    if (!decision.accepted) {
      result.accepted = accepted;
      result.next_token = decision.token;
      return result;
    }
  }
  result.accepted = accepted;
  result.status = qo_sample_distribution(
      target[draft_count], target_counts[draft_count],
      qo_counter_uniform(seed, position + accepted, 300u, 0u),
      &result.next_token);
  return result;
}

/* ---- synthetic inputs --------------------------------------------------------------- */

uint64_t qo_mix64(uint64_t seed, uint64_t index) {
  return splitmix64(seed ^ (index * 0x9e3779b97f4a7c15ull + 0x632be59bd9b4e019ull));
}

double qo_uniform01(uint64_t seed, uint64_t index) {
  return ((double)(qo_mix64(seed, index) >> 11) + 0.5) *
         (1.0 / 9007199254740992.0);
}

float qo_normal(uint64_t seed, uint64_t index) {
  const double u1 = qo_uniform01(seed, 2u * index);
  const double u2 = qo_uniform01(seed, 2u * index + 1u);
  return (float)(sqrt(-2.0 * log(u1)) * cos(6.283185307179586 * u2));
}
