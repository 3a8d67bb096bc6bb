// AddressSanitizer / UndefinedBehaviorSanitizer run of the library's host-only arithmetic: the plan, offsets and
// typed-piece tables of the streaming decode kernel (csrc/k_flow.hip, included as source; only its host functions run)
// and the synthetic-weight quantizers (csrc/synth.cpp).  No GPU call is made.  Every table entry is checked against the
// stream's bounds, which is what a wrong offset on the device would break.  Built and run by tests/test_sanitizers.py
// (hipcc with the sanitizers on the host side only).
#include "../../llama2.jl_amd/csrc/k_flow.hip"
#include "../../llama2.jl_amd/csrc/synth.cpp"

#include <stdio.h>

#include <string>
#include <vector>

static int fails = 0;
#define EXPECT(c)                                                 \
    do {                                                          \
        if (!(c)) {                                               \
            printf("line %d: %s\n", __LINE__, #c);                \
            fails++;                                              \
        }                                                         \
    } while (0)

static void check_shape(int dim, int hidden, int n_layers, int n_heads, int n_kv, int vocab, int seq_len, const int *layer7,
                        int cls_type, int kv16, bool expect_fit) {
    const int grid = 256;
    FlowArgs a{};
    a.dim = dim, a.hidden = hidden, a.n_layers = n_layers, a.n_heads = n_heads, a.n_kv_heads = n_kv;
    a.hs = dim / n_heads, a.kv_dim = a.hs * n_kv, a.seq_len = seq_len, a.vocab = vocab, a.kv16 = kv16;
    std::vector<int> types;
    for (int l = 0; l < n_layers; l++)
        for (int k = 0; k < 7; k++) types.push_back(layer7[k]);
    std::string why;
    const bool fit = k_flow_plan(a, types.data(), (int)types.size(), cls_type, grid, &why);
    EXPECT(fit == expect_fit);
    if (!fit) {
        EXPECT(!why.empty());
        return;
    }
    if (a.f32) return;  // no streams
    const FlowGeom g4[4] = {a.qkv, a.wo, a.w13, a.w2};
    for (int k = 0; k < 4; k++) {
        // every logical row has an owner, and the wavefronts' runs tile a workgroup's pieces exactly
        int64_t rows = 0;
        for (int wg = 0; wg < grid; wg++) {
            const int n = flow_n_local(g4[k], wg);
            rows += n;
            int pieces = 0;
            for (int w = 0; w < FLOW_NW; w++) {
                EXPECT(flow_wave_start(g4[k], wg, w) == pieces);
                pieces += flow_wave_pieces(g4[k], wg, w);
            }
            EXPECT(pieces == flow_wg_pieces(g4[k], wg));
            EXPECT(flow_half(g4[k]) ? pieces * 2 == n * flow_half(g4[k]) : pieces == n * g4[k].ppr);
            EXPECT(n <= FLOW_MAX_ROWS && pieces <= FLOW_MAX_PIECES / 4);
            if (flow_half(g4[k])) {
                // rows that end inside a piece: the pieces of a pair of rows hold every super-block of both rows once
                const int nb = 4 * flow_half(g4[k]);
                EXPECT(nb * 256 == dim && n % 2 == 0 && flow_half(g4[k]) % 2 == 1);
                std::vector<char> seen((size_t)n * nb, 0);
                for (int j = 0; j < pieces; j++) {
                    const int lr = flow_piece_row(g4[k], j), part = j % flow_half(g4[k]);
                    for (int b = 0; b < 8; b++) {
                        const int pb = 8 * part + b, odd = pb >= nb, blk = pb - odd * nb;
                        EXPECT(lr + odd < n && blk < nb);
                        EXPECT(!seen[(size_t)(lr + odd) * nb + blk]);
                        seen[(size_t)(lr + odd) * nb + blk] = 1;
                    }
                }
                for (char c : seen) EXPECT(c);
            }
        }
        EXPECT(rows == g4[k].n_rows);
    }
    if (a.mixed) {
        FlowTypedTables t;
        k_flow_typed_tables(a, types.data(), cls_type, grid, t);
        EXPECT(t.wave_off.size() == (size_t)grid * FLOW_NW && t.piece_off.size() == t.piece_tag.size());
        const int cls_piece = cls_type == L2H_TYPE_Q6_K ? FLOW_Q6_PIECE : FLOW_SLOT;
        for (size_t wi = 0; wi < t.wave_off.size(); wi++) {
            const int wg = (int)(wi / FLOW_NW), w = (int)(wi % FLOW_NW);
            const int64_t end = wi + 1 < t.wave_off.size() ? t.wave_off[wi + 1] : t.total - 4096;
            const int64_t first = t.piece_base[wi], last = wi + 1 < t.piece_base.size() ? t.piece_base[wi + 1] : (int64_t)t.piece_off.size();
            int64_t at = 0;
            for (int64_t e = first; e < last; e++) {
                const int ty = t.piece_tag[(size_t)e] & 0xFF;
                EXPECT(ty >= 0 && ty <= 2);
                EXPECT(t.piece_off[(size_t)e] == at);  // pieces lie back to back in consumption order
                at += flowm_piece_bytes(ty);
                // the tag names the type of the piece FLOWM_D places on (3: there is none)
                const int nxt = t.piece_tag[(size_t)e] >> 8;
                EXPECT(e + FLOWM_D < last ? nxt == (t.piece_tag[(size_t)(e + FLOWM_D)] & 0xFF) : nxt == 3);
            }
            EXPECT(t.cls_off[wi] == at);
            at += (int64_t)flow_wave_pieces(a.cls, wg, w) * cls_piece;
            EXPECT(t.wave_off[wi] + at <= end);
            EXPECT(t.wave_off[wi] % 256 == 0);
        }
    } else {
        std::vector<int64_t> off;
        const int64_t total = k_flow_offsets(a, cls_type, grid, off);
        EXPECT(off.size() == (size_t)grid * FLOW_NW);
        const int cls_piece = cls_type == L2H_TYPE_Q6_K ? FLOW_Q6_PIECE : FLOW_SLOT;
        for (size_t wi = 0; wi < off.size(); wi++) {
            const int wg = (int)(wi / FLOW_NW), w = (int)(wi % FLOW_NW);
            const int64_t end = wi + 1 < off.size() ? off[wi + 1] : total - 4096;
            const int64_t ring = (int64_t)n_layers * flow_layer_bytes(g4, wg, w, 4);
            const int64_t regs = (int64_t)n_layers * flow_layer_regs(g4, wg, w, 4) * FLOW_SLOT;
            EXPECT(flow_reg_base(g4, a.cls, cls_piece, n_layers, wg, w) == ring + (int64_t)flow_wave_pieces(a.cls, wg, w) * cls_piece);
            EXPECT(off[wi] + flow_reg_base(g4, a.cls, cls_piece, n_layers, wg, w) + regs <= end);
            EXPECT(off[wi] % 256 == 0);
        }
    }
    // logical row -> (tensor, row): a bijection onto the tensors' rows (both RoPE layouts, head sizes that are not powers of two)
    for (int neox = 0; neox < 2; neox++) {
        std::vector<char> seen((size_t)dim + 2 * a.kv_dim, 0);
        for (int L = 0; L < dim + 2 * a.kv_dim; L++) {
            int seg, row;
            flow_row_src(0, L, dim, a.kv_dim, a.hs, neox, seg, row, true);
            const int at = seg == 0 ? row : (seg == 1 ? dim + row : dim + a.kv_dim + row);
            EXPECT(seg >= 0 && seg <= 2 && row >= 0 && row < (seg == 0 ? dim : a.kv_dim));
            EXPECT(!seen[(size_t)at]);
            seen[(size_t)at] = 1;
        }
    }
}

int main() {
    const int q4[7] = {12, 12, 12, 12, 12, 12, 12}, q5m[7] = {13, 13, 13, 13, 13, 14, 13}, mix[7] = {12, 12, 13, 12, 12, 14, 12},
              f32[7] = {0, 0, 0, 0, 0, 0, 0}, bad[7] = {12, 12, 12, 12, 12, 12, 13};
    check_shape(4096, 14336, 32, 32, 8, 128256, 512, q4, 14, 0, true);    // the headline model
    check_shape(4096, 14336, 32, 32, 8, 128256, 4096, q5m, 14, 0, true);  // q5_K_M mix: typed pieces
    check_shape(4096, 14336, 4, 32, 8, 128256, 512, mix, 12, 0, true);    // q4_K classifier behind typed pieces
    check_shape(3072, 8192, 32, 32, 32, 32064, 4096, q4, 12, 0, true);    // Phi-3: a piece and a half per row, head size 96
    check_shape(3072, 8192, 2, 32, 32, 32064, 4096, q4, 12, 1, true);     // the same with an fp16 cache
    check_shape(2048, 4096, 3, 16, 4, 1000, 160, q4, 14, 0, false);       // q6_K classifier needs 4096
    check_shape(2048, 4096, 3, 16, 4, 1000, 160, q4, 12, 0, true);
    check_shape(1536, 2048, 2, 16, 16, 999, 96, q4, 12, 0, true);         // a quarter below 2048: padded rows
    check_shape(3072, 8192, 2, 32, 8, 32064, 512, mix, 12, 0, true);      // halves with typed pieces and grouped heads
    check_shape(1024, 2048, 2, 16, 16, 999, 96, q4, 12, 0, false);        // half below: refused
    check_shape(512, 1376, 8, 8, 8, 32000, 1024, f32, 0, 0, true);        // llama2.c shape
    check_shape(4096, 14336, 2, 32, 8, 32000, 512, bad, 14, 0, false);    // w1 and w3 of different types
    check_shape(4096, 14336, 2, 32, 8, 32000, 40000, q4, 14, 0, false);   // cache too long for the attention area
    // synthetic weights: every quantizer over a few thousand values, odd thread counts
    std::vector<float> x(256 * 37);
    for (int t = 1; t <= 5; t += 2) {
        EXPECT(l2h_synth_normal(7, 3, 11, (int64_t)x.size(), 0.02f, x.data(), t) == 0);
        for (int type : {12, 13, 14}) {
            const int64_t bb = type == 12 ? 144 : (type == 13 ? 176 : 210);
            std::vector<uint8_t> out((size_t)(x.size() / 256) * (size_t)bb);
            EXPECT(l2h_quantize_weights(type, x.data(), (int64_t)x.size(), out.data(), t) == 0);
        }
    }
    EXPECT(l2h_quantize_weights(12, x.data(), 100, x.data(), 1) != 0);
    if (fails) {
        printf("%d checks failed\n", fails);
        return 1;
    }
    puts("host arithmetic: sanitizers silent, tables consistent");
    return 0;
}
