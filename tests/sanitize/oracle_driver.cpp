// Host-only sanitizer run of the CPU oracle: built together with oracle/ellm_oracle.cpp under
// -fsanitize=address,undefined by tests/test_abi_layout.py and run once.  Every buffer is a
// heap allocation of exactly the size the call is entitled to touch, so a read or write one
// element out of range (a wrong stride, an off-by-one position) aborts the run.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

extern "C" {
struct ellm_oracle_attn {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  float* lse;
  size_t batch_capacity, attention_head_num, kv_head_num, head_size;
  size_t kv_strides[4];
  float inverse_sqrt_head;
  int dtype;
};
int ellm_oracle_attention_run(const ellm_oracle_attn* op, size_t position_index, size_t position_interval,
                              size_t batch_size, const uint32_t* positions, size_t cpu_num, size_t thread_id);
double ellm_oracle_attention_run_threads(const ellm_oracle_attn* op, size_t position_index,
                                         size_t position_interval, size_t batch_size, const uint32_t* positions,
                                         size_t n_threads, int pin, size_t repeats);
double ellm_oracle_attention_rows_threads_ex(const ellm_oracle_attn* op, size_t position_index,
                                             const uint32_t* positions, const uint32_t* rows, size_t n_rows,
                                             void* out_rows, float* lse_rows, size_t n_threads, int pin);
int ellm_oracle_kv_append_norm_rope(void* k_cache, void* v_cache, size_t kv_heads, size_t capacity,
                                    size_t head_size, size_t position_index, size_t n_tokens, size_t batch_size,
                                    const void* k_src, const void* v_src, size_t src_batch_pitch, const void* rope,
                                    size_t rope_positions, float eps, const uint32_t* positions, int dtype);
int ellm_oracle_matmul3(const void* hidden, const void* wq, const void* wk, const void* wv, void* q_state,
                        void* k_state, void* v_state, const void* rope, size_t rope_pos_stride,
                        size_t rope_head_stride, size_t rope_elems, size_t k, size_t batch_pitch, size_t batch_size,
                        size_t q_heads, size_t kv_heads, size_t head, const size_t* kv_strides, size_t capacity,
                        size_t position_index, size_t interval, const uint32_t* positions, float eps, int dtype);
void ellm_oracle_matmul_add(const void* a, const void* b_nt, const void* residual, void* output, size_t n, size_t k,
                            size_t batch_pitch, size_t batch_size, size_t interval, int dtype);
long ellm_oracle_schedule_calls(size_t prompt_begin, size_t prompt_end, size_t chunk, size_t generation_end,
                                size_t* positions, size_t* intervals, size_t capacity);
uint16_t ellm_oracle_f32_to_f16(float f);
uint16_t ellm_oracle_f32_to_bf16(float f);
}

static uint32_t g_state = 12345u;
static float rnd() {  // small deterministic values in (-1, 1)
  g_state = g_state * 1664525u + 1013904223u;
  return (float)((int)(g_state >> 8) % 2001 - 1000) / 1000.0f;
}
// exactly n 16-bit elements on the heap
static uint16_t* halves(size_t n, int dtype) {
  uint16_t* p = (uint16_t*)malloc(n * sizeof(uint16_t));
  for (size_t i = 0; i < n; ++i) p[i] = dtype == 0 ? ellm_oracle_f32_to_f16(rnd()) : ellm_oracle_f32_to_bf16(rnd());
  return p;
}
#define REQUIRE(x) do { if (!(x)) { printf("FAILED: %s (line %d)\n", #x, __LINE__); return 1; } } while (0)

int main() {
  const size_t D = 128;
  for (int dtype = 0; dtype < 2; ++dtype) {
    // attention: chunk of 5 tokens from position 3, 2 of 3 sequences, 4 query / 2 kv heads, cache of 8
    const size_t S = 5, bcap = 3, b = 2, hq = 4, hkv = 2, cap = 8, p0 = 3;
    uint16_t* q = halves(S * bcap * hq * D, dtype);
    uint16_t* k = halves(b * hkv * cap * D, dtype);   // only the sequences that are run
    uint16_t* v = halves(b * hkv * cap * D, dtype);
    uint16_t* out = halves(S * bcap * hq * D, dtype);
    float* lse = (float*)malloc(S * bcap * hq * sizeof(float));
    ellm_oracle_attn op = {q, k, v, out, lse, bcap, hq, hkv, D, {hkv * cap * D, cap * D, D, 1}, 0.0883883f, dtype};
    REQUIRE(ellm_oracle_attention_run(&op, p0, S, b, nullptr, 1, 0) == 0);
    REQUIRE(ellm_oracle_attention_run_threads(&op, p0, S, b, nullptr, 3, 1, 2) >= 0.0);
    // single-token step with per-sequence positions, the last one at the cache's last row
    const uint32_t positions[2] = {2, (uint32_t)cap - 1};
    REQUIRE(ellm_oracle_attention_run(&op, 0, 1, b, positions, 2, 1) == 0);
    const uint32_t rows[6] = {0, 0, 3, 0, 1, 0};
    uint16_t* out_rows = halves(2 * D, dtype);
    float lse_rows[2];
    REQUIRE(ellm_oracle_attention_rows_threads_ex(&op, 0, positions, rows, 2, out_rows, lse_rows, 2, 1) >= 0.0);
    // rejected arguments touch nothing
    REQUIRE(ellm_oracle_attention_run(&op, 0, 1, bcap + 1, nullptr, 1, 0) == 1);
    REQUIRE(ellm_oracle_attention_run(&op, 0, 2, b, positions, 1, 0) == 1);

    // cache write with norm + rotation: 3 tokens ending at the last row; table of exactly cap rows
    const size_t n_tok = 3, pitch = 3;
    uint16_t* ks = halves(n_tok * pitch * hkv * D, dtype);
    uint16_t* vs = halves(n_tok * pitch * hkv * D, dtype);
    uint16_t* rope = halves(cap * D, dtype);
    REQUIRE(ellm_oracle_kv_append_norm_rope(k, v, hkv, cap, D, cap - n_tok, n_tok, b, ks, vs, pitch, rope, cap, 1e-6f,
                                            nullptr, dtype) == 0);
    REQUIRE(ellm_oracle_kv_append_norm_rope(k, v, hkv, cap, D, cap - n_tok + 1, n_tok, b, ks, vs, pitch, rope, cap,
                                            1e-6f, nullptr, dtype) == 1);

    // fused projection: K = 64, 2 tokens x 2 of 3 sequences, writing at the last two rows
    const size_t K = 64, T = 2;
    uint16_t* hid = halves(T * pitch * K, dtype);
    uint16_t* wq = halves(hq * D * K, dtype);
    uint16_t* wk = halves(hkv * D * K, dtype);
    uint16_t* wv = halves(hkv * D * K, dtype);
    uint16_t* qs = halves(T * pitch * hq * D, dtype);
    const size_t strides[4] = {hkv * cap * D, cap * D, D, 1};
    REQUIRE(ellm_oracle_matmul3(hid, wq, wk, wv, qs, k, v, rope, D, 0, cap * D, K, pitch, b, hq, hkv, D, strides, cap,
                                cap - T, T, nullptr, 1e-6f, dtype) == 0);
    REQUIRE(ellm_oracle_matmul3(hid, wq, wk, wv, qs, k, v, rope, D, 0, cap * D, K, pitch, b, hq, hkv, D, strides, cap,
                                cap - T + 1, T, nullptr, 1e-6f, dtype) == 1);
    // output projection + residual: n = 128, k = 64
    uint16_t* bn = halves(128 * K, dtype);
    uint16_t* res = halves(T * pitch * 128, dtype);
    uint16_t* o2 = halves(T * pitch * 128, dtype);
    ellm_oracle_matmul_add(hid, bn, res, o2, 128, K, pitch, b, T, dtype);

    for (void* p : {(void*)q, (void*)k, (void*)v, (void*)out, (void*)lse, (void*)out_rows, (void*)ks, (void*)vs,
                    (void*)rope, (void*)hid, (void*)wq, (void*)wk, (void*)wv, (void*)qs, (void*)bn, (void*)res,
                    (void*)o2})
      free(p);
  }
  // schedule: exactly as many slots as calls; one fewer must be refused without writing past the end
  size_t* pos = (size_t*)malloc(5 * sizeof(size_t));
  size_t* itv = (size_t*)malloc(5 * sizeof(size_t));
  REQUIRE(ellm_oracle_schedule_calls(0, 150, 64, 152, pos, itv, 5) == 5);
  REQUIRE(pos[2] == 128 && itv[2] == 22 && pos[4] == 151 && itv[4] == 1);
  size_t* pos4 = (size_t*)malloc(4 * sizeof(size_t));
  size_t* itv4 = (size_t*)malloc(4 * sizeof(size_t));
  (void)ellm_oracle_schedule_calls(0, 150, 64, 152, pos4, itv4, 4);
  free(pos); free(itv); free(pos4); free(itv4);
  printf("sanitizer run: ok\n");
  return 0;
}
