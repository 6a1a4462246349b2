// tzgemm_kernel.h -- host object of the tensor GEMM and its shape rule.
//
// Public surface of src/tzgemm_kernel.h of the reference: getTZGEMMGridDim and
// OriTZGEMMKernel(id, m, n, k) with parameters {&A, &B, &C, &M_GLOBAL, &N_GLOBAL,
// &K_GLOBAL} over process-lifetime global device buffers ori_wmma_{A,B,C}.  The
// tile count keeps the reference's unit (64x64 tiles) because that is what
// callers pass as ptb_end_block_pos; the gfx950 kernel groups 2x2 of them into
// its 128x128 macro tile internally.
//
// Differences: the global buffers grow on demand (the reference sizes them once,
// from the first shape it sees), and a second constructor binds caller-owned
// buffers, which is what the C entry points use.  The parameter list is the
// reference's six.  The shapes whose reduction is cut over several workgroups
// need a workspace (partial tiles and arrival counters); the library keeps one
// per output buffer C (tzgemmWorkspaceFor) and publishes the pair in a
// device-resident table in which the kernels look their C up.
#pragma once

#include <algorithm>
#include <vector>

#include "Kernel.h"
#include "Logger.h"
#include "header/tzgemm_header.h"

extern Logger logger;
extern long long MAX_ORI_WMMA_A;   // bytes currently allocated for each global buffer
extern long long MAX_ORI_WMMA_B;
extern long long MAX_ORI_WMMA_C;
extern bool gemm_malloced;
extern void *ori_wmma_A;           // f16 [M][K]
extern void *ori_wmma_B;           // f16 [N][K]
extern float *ori_wmma_C;          // f32 [M][N]

inline int tzgemmRoundDim(int x) { return (x < 128) ? 128 : (x / 128) * 128; }

// {M_GLOBAL, N_GLOBAL, K_GLOBAL, number of 64x64 tiles}
inline std::vector<int> getTZGEMMGridDim(int m, int n, int k)
{
    const int M_GLOBAL = tzgemmRoundDim(m);
    const int N_GLOBAL = tzgemmRoundDim(n);
    const int K_GLOBAL = tzgemmRoundDim(k);
    const int tiles = (M_GLOBAL / TZ_REF_TILE) * (N_GLOBAL / TZ_REF_TILE);
    return std::vector<int>{M_GLOBAL, N_GLOBAL, K_GLOBAL, tiles};
}

// Allocates / grows the global GEMM buffers so that an (M,N,K) problem fits, and
// fills A and B with seeded uniform[-1,1] halves the first time (the reference
// leaves them zero after cudaMemset; synthetic operands make the result checkable).
void ensureGlobalGemmBuffers(int M_GLOBAL, int N_GLOBAL, int K_GLOBAL);

// Workspace for GEMMs that write the buffer C: nullptr when the shape needs none, else a zeroed
// device buffer of at least tz_workspace_bytes(M, N, K) bound to C (or a larger one that replaces
// it), entered into the device table tz_ws_table where the kernels find it.  Launches that write
// the same C must not overlap anyway, so they can share it; launches on different C never do.
// The caller becomes a user of the binding until it calls tzgemmWorkspaceDone with the same
// arguments; a binding without users stays for the next kernel object on the same C and is taken
// out, least recently used first, when the table or the device memory such bindings may hold
// (512 bindings, 1 GiB) is needed for a new one.  Thread-safe.
void *tzgemmWorkspaceFor(const float *C, int M_GLOBAL, int N_GLOBAL, int K_GLOBAL);
void tzgemmWorkspaceDone(const float *C, int M_GLOBAL, int N_GLOBAL, int K_GLOBAL);
// bindings in the table, those with a user, device bytes they hold (any pointer may be null)
void tzgemmWorkspaceStats(int *bindings, int *in_use, long long *bytes);
// Frees every workspace after a device synchronisation.  Only when no kernel object that uses one
// is left.
void tzgemmReleaseWorkspaces();

class OriTZGEMMKernel : public Kernel {
public:
    OriTZGEMMKernel(int id, int m, int n, int k) : m(m), n(n), k(k)
    {
        this->Id = id;
        this->kernelName = "tzgemm";
        useGlobals = true;
        this->initParams();
    }
    // caller-owned operands; dimensions are still rounded by the same rule
    OriTZGEMMKernel(int id, int m, int n, int k, const void *A, const void *B, float *C)
        : m(m), n(n), k(k), A_(const_cast<void *>(A)), B_(const_cast<void *>(B)), C_(C)
    {
        this->Id = id;
        this->kernelName = "tzgemm";
        useGlobals = false;
        this->initParams();
    }
    ~OriTZGEMMKernel() override { dropWorkspace(); }

    void initParams() override
    {
        const std::vector<int> d = getTZGEMMGridDim(m, n, k);
        M_GLOBAL = d[0];
        N_GLOBAL = d[1];
        K_GLOBAL = d[2];
        ori_blks = d[3];
        dropWorkspace();   // of an earlier initParams
        if (useGlobals) ensureGlobalGemmBuffers(M_GLOBAL, N_GLOBAL, K_GLOBAL);
        tzgemmWorkspaceFor(useGlobals ? ori_wmma_C : C_, M_GLOBAL, N_GLOBAL, K_GLOBAL);
        ws_m = M_GLOBAL, ws_n = N_GLOBAL, ws_k = K_GLOBAL;

        launchGridDim = dim3(ori_blks, 1, 1);
        launchBlockDim = dim3(TZ_THREADS, 1, 1);
        kernelParams.clear();
        kernelParams.push_back(useGlobals ? (void *)&ori_wmma_A : (void *)&A_);
        kernelParams.push_back(useGlobals ? (void *)&ori_wmma_B : (void *)&B_);
        kernelParams.push_back(useGlobals ? (void *)&ori_wmma_C : (void *)&C_);
        kernelParams.push_back(&M_GLOBAL);
        kernelParams.push_back(&N_GLOBAL);
        kernelParams.push_back(&K_GLOBAL);
        this->smem = TZ_LDS_BYTES;
    }

    std::vector<int> getArgs() override { return std::vector<int>{m, n, k}; }
    // shapes with a 256 x 256 tile for every CU run the large-tile build of general_ptb_tzgemm
    // (same parameter list, same bits)
    const char *funcVariant() override { return tz_use_large(M_GLOBAL, N_GLOBAL, K_GLOBAL) ? "@large" : ""; }

    int m, n, k;
    int M_GLOBAL, N_GLOBAL, K_GLOBAL;
    int ori_blks;

protected:
    // as in the reference, the GEMM only ever runs in its GPTB or fused form
    void executeImpl(cudaStream_t) override
    {
        printf("should not execute ori tzgemm!\n");
        exit(1);
    }

private:
    void loadKernel() override {}
    // this object is no longer a user of the workspace bound to its output buffer (the global C may
    // have moved since: its bindings moved with it)
    void dropWorkspace()
    {
        if (ws_m) tzgemmWorkspaceDone(useGlobals ? ori_wmma_C : C_, ws_m, ws_n, ws_k);
        ws_m = ws_n = ws_k = 0;
    }
    int ws_m = 0, ws_n = 0, ws_k = 0;   // shape whose workspace this object holds a use of
    bool useGlobals;
    void *A_ = nullptr;
    void *B_ = nullptr;
    float *C_ = nullptr;
};
