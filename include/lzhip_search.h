/* C ABI of the callers directly above ForwardPipe::forward: input planes,
 * one full network evaluation (planes -> device -> heads -> un-rotated policy)
 * and a multi-threaded tree-search driver that exercises the backend the way
 * the engine's search does.  Plain pointers and sizes only. */
#ifndef LZHIP_SEARCH_C_H_INCLUDED
#define LZHIP_SEARCH_C_H_INCLUDED

#include <stdint.h>

#include "lzhip.h"

#ifdef __cplusplus
extern "C" {
#endif

#define LZHIP_BLACK 0
#define LZHIP_WHITE 1
#define LZHIP_EMPTY 2
#define LZHIP_PASS 361 /* moves are y*19+x, 361 = pass */

/* Head parameters as Network holds them (reference src/Network.h:166-183)
 * after the preprocessing of src/Network.cpp:351-352,568-576; same meaning as
 * the arguments of lzhip_push_heads.  Every entry point below that takes a
 * `heads` argument accepts NULL for "the parameters given to lzhip_push_heads"
 * (kept in host layout by the handle, so repeated calls do not re-pack them). */
typedef struct lzhip_head_weights {
    const float* bn_pol_mean;  /* [2]   conv bias folded in              */
    const float* bn_pol_scale; /* [2]   1/sqrt(var+1e-5)                 */
    const float* ip_pol_w;     /* [362][722]                             */
    const float* ip_pol_b;     /* [362]                                  */
    const float* bn_val_mean;  /* [1]                                    */
    const float* bn_val_scale; /* [1]                                    */
    const float* ip1_val_w;    /* [256][361]                             */
    const float* ip1_val_b;    /* [256]                                  */
    const float* ip2_val_w;    /* [256]                                  */
    const float* ip2_val_b;    /* [1]                                    */
} lzhip_head_weights;

/* Search parameters; lzhip_search_default_config fills the engine's defaults
 * (reference src/GTP.cpp:346-354, src/UCTNode.h:51, src/NNCache.h:44-47). */
typedef struct lzhip_search_config {
    int threads;       /* search threads (reference --threads)                    */
    int visits;        /* root visits per move (reference --visits)               */
    int moves;         /* moves of self-play to generate                          */
    int cache_size;    /* evaluation cache entries, 0 = no cache                  */
    int reuse_tree;    /* keep the chosen subtree between moves                   */
    int random_moves;  /* first N moves sampled in proportion to visits           */
    int virtual_loss;  /* 3                                                        */
    int device_heads;  /* 1: heads computed on the device (lzhip_forward_eval) instead
                          of on the search threads; needs lzhip_push_heads          */
    float puct;        /* 0.5                                                      */
    float logpuct;     /* 0.015                                                    */
    float logconst;    /* 1.7                                                      */
    float fpu_reduction; /* 0.25: first-play urgency reduction below the root      */
    float fpu_root_reduction; /* at the root; 0.25 (reference cfg_fpu_root_reduction,
                                 src/GTP.cpp:354, used at src/UCTNode.cpp:322-324)  */
    float softmax_temp;  /* 1.0                                                    */
    float komi;          /* 7.5                                                    */
    uint64_t seed;
} lzhip_search_config;

typedef struct lzhip_search_result {
    uint64_t playouts;      /* simulations that returned a value                   */
    uint64_t wasted;        /* simulations that met a node under expansion         */
    uint64_t halted;        /* simulations cut short by the halt at end of move    */
    uint64_t evals;         /* network evaluations sent to the backend             */
    uint64_t cache_lookups;
    uint64_t cache_hits;
    uint64_t nodes;         /* tree nodes created                                  */
    double seconds;         /* wall time of the search phases                      */
    double visits_per_s;    /* playouts / seconds                                  */
    int moves_played;
    int passes_at_end;      /* 2 when the game ended by two passes                 */
    float final_score;      /* black area minus white area minus komi              */
    lzhip_stats sched;      /* scheduler counters accumulated during the run       */
} lzhip_search_result;

/* Network::get_symmetry / symmetry_nn_idx_table (reference
 * src/Network.cpp:968-993, :518-531): board index read by NN index `idx`
 * under `symmetry` (0..7); -1 on bad arguments. */
int lzhip_symmetry_index(int symmetry, int idx);

/* Network::gather_features (reference src/Network.cpp:935-966).  `boards`
 * holds n_boards (1..8) positions of 361 bytes, newest first, each byte
 * LZHIP_BLACK / LZHIP_WHITE / LZHIP_EMPTY; to_move is the side to move now.
 * out [18][361]: planes 0-7 side to move, 8-15 opponent, 16 ones if black is
 * to move, 17 ones if white is. */
int lzhip_gather_features(const uint8_t* boards, int n_boards, int to_move, int symmetry,
                          float* out);

/* Network::get_output_internal (reference src/Network.cpp:811-864) for one
 * position: planes under `symmetry`, one blocking request through the
 * scheduler, heads on the calling thread, policy rotated back to board order.
 * policy [362] (index 361 = pass), *winrate in [0,1] for the side to move.
 * Thread-safe; returns LZHIP_EHALT while drained. */
int lzhip_get_output(lzhip_handle* h, const lzhip_head_weights* heads, const uint8_t* boards,
                     int n_boards, int to_move, int symmetry, float softmax_temp,
                     float* policy, float* winrate);

/* Network::get_output with Ensemble::AVERAGE (reference src/Network.cpp:762-775):
 * the mean over the eight symmetries of policy, pass probability and winrate.
 * The eight symmetric inputs are evaluated as device batches (one batch of 8
 * when max_batch >= 8) directly on the pipe, not through the request queue, so
 * drain() does not interrupt it; heads run on the calling thread. */
int lzhip_get_output_average(lzhip_handle* h, const lzhip_head_weights* heads,
                             const uint8_t* boards, int n_boards, int to_move,
                             float softmax_temp, float* policy, float* winrate);

/* Network::m_value_head_not_stm (reference src/Network.cpp:395-400): networks of
 * weights-file format 2 give the value for black instead of for the side to
 * move, and Network::get_output turns it round when white is to move
 * (src/Network.cpp:797-802).  With `on` non-zero lzhip_get_output,
 * lzhip_get_output_average and the search driver do the same; off by default.
 * Set it before evaluations start. */
int lzhip_set_value_head_not_stm(lzhip_handle* h, int on);

/* Network::benchmark (reference src/Network.cpp:128-149; the GTP command
 * `netbench`, src/GTP.cpp:1055-1069): `threads` threads evaluate the given
 * position, each time under a random symmetry and without the cache, until
 * `iterations` evaluations have been started; every evaluation is one request
 * through the scheduler with the heads on the calling thread, as in
 * lzhip_get_output.  *evaluations is the number done (up to threads - 1 more than
 * asked for, as in the reference), *seconds the wall time they took. */
int lzhip_netbench(lzhip_handle* h, const lzhip_head_weights* heads, const uint8_t* boards,
                   int n_boards, int to_move, int threads, int iterations, uint64_t seed,
                   int* evaluations, double* seconds);

int lzhip_search_default_config(lzhip_search_config* cfg);

/* Self-play from the empty board with cfg->threads search threads calling the
 * backend one position at a time, as UCTSearch::think does (reference
 * src/UCTSearch.cpp:237-286, :757-850): virtual loss, PUCT selection,
 * expansion by one network evaluation with a random symmetry, evaluation
 * cache, halt of outstanding requests when a move's visit budget is reached.
 * moves_out (may be NULL) receives up to moves_cap played moves. */
int lzhip_selfplay(lzhip_handle* h, const lzhip_head_weights* heads,
                   const lzhip_search_config* cfg, lzhip_search_result* result,
                   int* moves_out, int moves_cap);

/* Go rules used by the driver, exposed for checking: replays `moves` (each
 * legal for the side to move, or LZHIP_PASS) from the empty board.  Outputs
 * (each may be NULL): stones [361], legal [362] for the side to move
 * (FastState::is_move_legal, reference src/FastState.cpp:76-83), *ko_point
 * (-1 if none), *superko (the last move repeated an earlier position,
 * reference src/KoState.cpp:51-58), *score (FastBoard::area_score, reference
 * src/FastBoard.cpp:260-296, with the given komi).  Returns LZHIP_EINVAL at
 * the first illegal move. */
int lzhip_board_replay(const int* moves, int n_moves, float komi, uint8_t* stones,
                       uint8_t* legal, int* ko_point, int* superko, float* score);

#ifdef __cplusplus
}
#endif
#endif
