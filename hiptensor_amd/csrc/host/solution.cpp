#include "solution.hpp"

#include <algorithm>
#include <cmath>

namespace hipta
{
    static uint64_t mix(uint64_t h, uint64_t v)
    {
        // 64-bit variant of the boost-style combine the reference uses for its solution
        // ids (library/src/include/hash.hpp:50-58)
        return h ^ (v + 0x9e3779b97f4a7c15ull + (h << 6) + (h >> 2));
    }

    SolutionRegistry::SolutionRegistry()
    {
        for(int cls = 0; cls < HIPTK_NUM_CLASSES; cls++)
        {
            const int n = hiptk_tile_count(cls);
            for(int t = 0; t < n; t++)
            {
                hiptk_tile_info_t ti;
                if(hiptk_tile_info(cls, t, &ti) != HIPTK_OK)
                    continue;
                Solution s;
                s.cls       = cls;
                s.tile_id   = t;
                s.bp        = ti.bp;
                s.bq        = ti.bq;
                s.bk        = ti.bk;
                s.threads   = ti.threads;
                s.lds_bytes = ti.lds_bytes;
                s.direct    = ti.k_multiple > 0;
                s.mfma_k    = ti.mfma_k;
                s.name      = ti.name;
                uint64_t h  = 0x68697074656e73ull;
                for(uint64_t x : {(uint64_t)cls, (uint64_t)t, (uint64_t)ti.bp, (uint64_t)ti.bq, (uint64_t)ti.bk})
                    h = mix(h, x);
                s.uid = h;
                mAll.push_back(s);
            }
        }
    }

    const SolutionRegistry& SolutionRegistry::get()
    {
        static const SolutionRegistry r;
        return r;
    }

    std::vector<const Solution*> SolutionRegistry::forClass(int cls) const
    {
        std::vector<const Solution*> out;
        for(const Solution& s : mAll)
            if(s.cls == cls)
                out.push_back(&s);
        return out;
    }

    const Solution* SolutionRegistry::byUid(uint64_t uid) const
    {
        for(const Solution& s : mAll)
            if(s.uid == uid)
                return &s;
        return nullptr;
    }

    bool solution_fits(const Solution& s, const GemmView& v)
    {
        if(s.cls != v.cls)
            return false;
        hiptk_problem_t p{};
        p.cls     = v.cls;
        p.tile_id = s.tile_id;
        p.x_kfast = v.x_kfast;
        p.y_kfast = v.y_kfast;
        p.x_vec   = v.x_vec;
        p.y_vec   = v.y_vec;
        p.k_affine = v.k_affine;
        p.P        = v.P;
        p.Q        = v.Q;
        p.K        = v.K;
        p.shift_p  = v.shift_p;
        p.shift_q  = v.shift_q;
        p.xy_aligned = v.xy_aligned;
        p.x_max_off  = (int32_t)v.x_max_off;
        p.y_max_off  = (int32_t)v.y_max_off;
        return hiptk_kernel_available(&p) != 0;
    }

    double class_flops_per_clk_cu(int cls)
    {
        switch(cls)
        {
        case HIPTK_F16:
        case HIPTK_BF16:
        case HIPTK_F32_AS_F16:
        case HIPTK_F32_AS_BF16: return 4096.0;
        case HIPTK_F64:
        case HIPTK_C64: return 128.0;
        default: return 256.0;
        }
    }

    double class_flops_per_mac(int cls)
    {
        return (cls == HIPTK_C32 || cls == HIPTK_C64) ? 8.0 : 2.0;
    }

    int class_acc_bytes(int cls)
    {
        switch(cls)
        {
        case HIPTK_F64:
        case HIPTK_C32: return 8;
        case HIPTK_C64: return 16;
        default: return 4;
        }
    }

    namespace
    {
        // Measured on MI355X with this library's kernels at the device's sustained clock and
        // with random operands, as fractions of the class's nominal MFMA peak per CU
        // (2.4 GHz x flop/clk/CU): `alone` is what one workgroup of the tile sustains when it
        // has a CU to itself (latency bound), `full` what a CU sustains with as many of them
        // resident as fit.  For orientation, a loop of nothing but MFMA instructions on random
        // operands sustains 0.65 (f16), 0.71 (bf16), 0.98 (f32) and 0.86 (f64) of nominal.
        struct TileRate
        {
            double alone, full;
        };

        TileRate tile_rate(int cls, int area)
        {
            switch(cls)
            {
            case HIPTK_F16:
            case HIPTK_BF16:
            case HIPTK_F32_AS_F16:
            case HIPTK_F32_AS_BF16:
                return area >= 65536   ? TileRate{0.44, 0.44}
                       : area >= 49152 ? TileRate{0.40, 0.40}
                       : area >= 32768 ? TileRate{0.38, 0.38}
                       : area >= 16384 ? TileRate{0.34, 0.315}
                                       : TileRate{0.107, 0.21};
            case HIPTK_F64:
                // (the 64 x 64 tile runs on eight waves, 16 x 32 outputs each: alone on a CU it reaches 0.64 of
                // nominal on 1024^3 f64 against 0.53 on four waves; 1920^2 x 768: 104.9 against 108.1 us)
                // (many short tiles per CU, 4096^2 x 512: 128 x 128 258-265 us on k-contiguous operands, 296-314 on
                // row-contiguous ones (estimate_us), 64 x 64 269-273, where the direct-load 64 x 64 tile, whose prologue
                // nothing overlaps, needs 280-294)
                return area >= 16384 ? TileRate{0.83, 0.83} : TileRate{0.60, 0.80};
            case HIPTK_C64:
                // (2048^2 x 1024: 527 us on either tile; 1920^2 x 768: 406 us on 900 tiles of 64 x 64, 375 us on
                // 3600 of 32 x 32; 512^3, one tile per CU: 74.8 us on 64 of the one, 26.6 us on 256 of the other)
                // (1024^2 x 512, four 32 x 32 tiles per CU: 75.2 us; 512^3 in two slices 28.7)
                return area >= 4096 ? TileRate{0.70, 0.82} : TileRate{0.50, 0.78};
            // (128 x 128 on 4096 x 4096 x 512, four tiles per CU: complex f32 535 us, f32 140.5 us; complex f32 on
            // 64 x 64: 1024^2 x 512 in one pass 50.7 us, 3072 x 1024 x 1024 203.6 us)
            case HIPTK_C32: return area >= 16384 ? TileRate{0.84, 0.86} : TileRate{0.62, 0.82};
            // (f32 128 x 128, one tile per CU: 1920^2 x 768 66 us, 2048^2 x 1024 85 us)
            default: return area >= 16384 ? TileRate{0.66, 0.85} : TileRate{0.36, 0.66};
            }
        }
    }

    double estimate_us(const Solution& s, const GemmView& v, int split, const DeviceModel& dev)
    {
        const double tiles  = std::ceil((double)v.P / s.bp) * std::ceil((double)v.Q / s.bq);
        const double ktiles = std::ceil((double)v.K / s.bk);
        const double kper   = std::ceil(ktiles / split) * s.bk;
        // workgroups that fit on one CU at a time: bound by LDS and by 16 wavefronts per CU
        // (kernels are compiled for at least two waves per SIMD, none for more than four)
        int resident = std::max(1, std::min({4, dev.lds_per_cu / std::max(1, s.lds_bytes), 1024 / std::max(64, s.threads)}));
        const double wgs     = tiles * split;
        const double per_cu  = std::ceil(wgs / dev.cus); // workgroups the busiest CU runs
        const double sharing = std::min<double>(resident, per_cu);
        TileRate     r       = tile_rate(v.cls, s.bp * s.bq);
        double round_extra_us = 0.0;
        if(v.cls == HIPTK_F64 && s.bp * s.bq >= 16384 && !(v.x_kfast && v.y_kfast))
            r = TileRate{0.74, 0.74};
        if(class_flops_per_clk_cu(v.cls) == 4096.0 && s.direct && s.bk == 64)
        {
            // The 256 x 256 tile on 16 x 16 x 32 MFMAs whose operand tiles are loaded straight into LDS in K tiles of
            // 64 (four waves).  4096^3 f16 scale, one device: both operands k-contiguous 98.5 us (main loop 84.2,
            // prologue 1.5, epilogue 7.9) against 108.8 on the same loop with 32 x 32 x 16 MFMAs and 121.0 on the
            // eight-wave staged tile; both row-contiguous 105.5 against 114.7 on the 32 x 32 x 16 direct-load tile of
            // K tiles of 32 (bf16 bilinear 99.2 against 107.0).
            const double f = (v.x_kfast && v.y_kfast) ? 1.33 : (v.x_kfast || v.y_kfast) ? 1.28 : 1.235;
            r.alone *= f;
            r.full *= f;
            round_extra_us = 6.5;
        }
        else if(class_flops_per_clk_cu(v.cls) == 4096.0 && s.direct && s.bk == 32 && s.mfma_k == 32)
        {
            // The 256 x 192 tile on 16 x 16 x 32 MFMAs that reads its k offsets from tables and loads K tiles of 32 into
            // a ring of four stages.  Rank-6 benchmark layout (5376 x 6912 x 4080 f16 bilinear, three rounds of tiles,
            // X row-contiguous in runs of 64 bytes, Y k-contiguous in runs of 16, staged chunk-major): 265 us against
            // 300 on the 32 x 32 x 16 tile below (main loop of a round 67 against 80 us, epilogue 16 and 17.5).
            const double f = (v.x_kfast && v.y_kfast) ? 1.085 : (v.x_kfast || v.y_kfast) ? 1.225 : 1.36;
            r.alone *= f;
            r.full *= f;
            round_extra_us = 5.0;
        }
        else if(class_flops_per_clk_cu(v.cls) == 4096.0 && s.threads == 256 && s.bp * s.bq >= 49152 && s.bk == 32)
        {
            // The 256 x 256 and 256 x 192 tiles whose operand tiles are loaded straight into LDS (four waves,
            // K in steps of 32): a faster main loop, but one workgroup has the CU to itself, so nothing
            // overlaps its prologue and epilogue.  Fitted to 4096 x 4096 x K, one round of 256 x 256 tiles, f16
            // scale, against the eight-wave tile (us at K = 512 / 1024 / 2048 / 4096):
            //   both operands row-contiguous  25.4 / 38.8 / 62.2 / 110.1  against  23.9 / 37.0 / 64.9 / 121.3
            //   one of them k-contiguous      26.5 / 40.2 / 64.5 / 113.3  against  21.8 / 36.7 / 62.9 / 115.6
            //   both k-contiguous             25.8 / 40.0 / 65.2 / 118.8  against  21.6 / 35.3 / 60.8 / 112.0
            // i.e. 23.4 / 24.4 / 26.8 us per 1024 of K against 28.1 / 26.4 / 25.6, and 15.4 against 8.8 us that do
            // not depend on K; four rounds (8192 x 8192 x 512): 103.3 against 85.8 us.
            const double f = (v.x_kfast && v.y_kfast) ? 0.955 : (v.x_kfast || v.y_kfast) ? 1.08 : 1.20;
            r.alone *= f;
            r.full *= f;
            round_extra_us = 6.5;
        }
        else if(class_flops_per_clk_cu(v.cls) == 4096.0 && s.threads == 256 && s.bp * s.bq >= 49152)
        {
            // the four-wave form of the 256 x 256 tile (one wave per SIMD): level with the
            // eight-wave form over a long K without C, behind it in the epilogue that reads C
            // and over a short K, and wherever an operand is contiguous along k (4096^3 f16 scale,
            // both operands k-contiguous: 126.3 us against 120.5 on eight waves; one of them: 126.3
            // against 122-124.6)
            const double f = kper / s.bk < 24 ? 0.9 : v.bilinear ? 0.95 : (v.x_kfast || v.y_kfast) ? 0.96 : 1.005;
            r.alone *= f;
            r.full *= f;
        }
        if(s.direct && class_flops_per_clk_cu(v.cls) != 4096.0)
        {
            // The 32/64-bit 64 x 64 tiles whose operand tiles are loaded straight into LDS (four waves, three to
            // four workgroups per CU): slopes of 1024 x 1024 x K (one workgroup per CU) and 2048 x 2048 x K scans
            const bool big = s.bp * s.bq >= 4096; // 64 x 64, or 32 x 32 with the waves splitting K
            const bool kf  = v.x_kfast && v.y_kfast; // 16-byte vectors of k: shorter runs in memory
            switch(v.cls)
            {
            // (the 32 x 32 tile reads twice the operand bytes per flop: 1024^2 x 2048 f32 41.8 against 38.1 us,
            // 512 x 2048 x 4096 78.6 against 68.8; level with the 64 x 64 tile in f64 and c32 on row-contiguous
            // operands.  k-contiguous operands, 2048^2 x 1024 on 64 x 64: f32 74.8 us, f64 132.2, c32 244.3; on
            // 32 x 32 a wave's runs are 64 bytes a row and K tile: 1024^2 x 2048 f64 125 against 70.7 us)
            case HIPTK_F32: r = big ? (kf ? TileRate{0.75, 0.78} : TileRate{0.81, 0.89}) : (kf ? TileRate{0.55, 0.60} : TileRate{0.65, 0.70}); break;
            // (one operand k-contiguous, 1024^2 x 2048 f64 on 32 x 32: 82.9 against 70.8 us)
            case HIPTK_F64:
                r = big ? (kf ? TileRate{0.84, 0.88} : TileRate{0.82, 0.90})
                        : (kf ? TileRate{0.45, 0.50} : (v.x_kfast || v.y_kfast) ? TileRate{0.62, 0.66} : TileRate{0.82, 0.90});
                break;
            case HIPTK_C32: r = big ? (kf ? TileRate{0.88, 0.90} : TileRate{0.90, 0.91}) : (kf ? TileRate{0.85, 0.88} : TileRate{0.90, 0.91}); break;
            // (complex f64, one element per vector: 2048^2 x 1024 478 us on 64 x 64 against 525 staged, 1024^2 x 512 71.9;
            // on 32 x 32 tiles 512^3, one workgroup per CU, 24.0 us (28.7 on the staged tile in two slices); 1024^2 x 512,
            // four per CU, 92.7)
            case HIPTK_C64: r = big ? TileRate{0.85, 0.91} : TileRate{0.85, 0.70}; break;
            default: break;
            }
            // ... whose prologue (tables, then the first tiles' flight) and epilogue nothing overlaps when a
            // CU runs one or two rounds of them: 2048 x 2048 x K f32 fits 13.9 us + 60.5 us per 1024 of K
            // (256^3 f32: one pass 9.2-9.8 us, four slices of four K tiles 7.8-8.1 us with the reduction: a
            // slice shorter than the ring has less in flight to wait for); the 32 x 32 tile adds its partial
            // tiles through LDS (640^2 x 64 f32: 8.4 us against 6.3 on 64 x 64 tiles)
            // (k-contiguous: 8.6 against 6.5 us)
            // (complex f64 is "k-contiguous" on every layout: one element per vector)
            const bool short_runs = (v.x_kfast || v.y_kfast) && v.cls != HIPTK_C64;
            round_extra_us        = 2.0 * std::min(1.0, kper / s.bk / 16.0) + (big ? 0.0 : short_runs ? 2.5 : 1.0);
        }
        if(class_max_vec(v.cls) > 1)
        {
            // narrower gathers are issue bound: measured on 2040^3 f16 problems whose runs
            // admit 16 / 8 / 4 / 2 bytes per load: 456 / 395 / 209 / 114 TFLOP/s
            // (16-bit classes); the f32 kernels with 4-byte gathers reach 0.75-0.79 of their 16-byte
            // form (4845 x 4845 x 1001: 86 against 108 TFLOP/s; 1965 x 1965 x 1001: 115 against 86 us)
            const int    bytes = std::min(v.x_vec, v.y_vec) * v.elem_bytes;
            const bool   wide  = class_max_vec(v.cls) != 8;
            const double f     = bytes >= 16 ? 1.0 : bytes >= 8 ? 0.87 : wide ? 0.77 : bytes >= 4 ? 0.45 : 0.25;
            r.alone *= f;
            r.full *= f;
        }
        // (a workgroup that has its CU to itself runs at `alone`, which for waves that never meet at a barrier can
        // be above what two such workgroups reach together)
        const double frac     = sharing <= 1.0 ? r.alone : std::min(sharing * r.alone, r.full);
        const double flops_wg = class_flops_per_mac(v.cls) * (double)s.bp * s.bq * kper;
        const double cu_rate  = class_flops_per_clk_cu(v.cls) * dev.clock_ghz * 1e3; // flop / us
        double       us       = per_cu * flops_wg / (frac * cu_rate);
        // memory floor: every operand once (+ C and D)
        const double bytes = ((double)v.P * v.K + (double)v.Q * v.K + (double)v.P * v.Q * (v.bilinear ? 2 : 1))
                             * v.elem_bytes;
        us = std::max(us, bytes / (dev.hbm_gbs * 1e3 * 0.6));
        // split-K slices of different tiles share nothing in time: every workgroup's operand panels come through
        // the fabric (256 x 256 x 65536 f16 in 32 slices: 16 tiles of 64 x 64 move 2.7e8 B for 6.7e7 algorithmic
        // and take 40.5 us, 4 tiles of 128 x 128 move half of that and take 33.4)
        if(split > 1)
            us = std::max(us, tiles * (double)(s.bp + s.bq) * (double)v.K * v.elem_bytes / (dev.hbm_gbs * 1e3 * 1.4));
        // launch, and prologue + epilogue of every round of workgroups on a CU
        // (a workgroup's epilogue moves its output tile, and C, at about 30 GB/s per CU)
        const double tile_io = (double)s.bp * s.bq * v.elem_bytes * (v.bilinear ? 2.0 : 1.0) / 30e3;
        us += 2.0 + (1.0 + tile_io + round_extra_us) * std::ceil(per_cu / sharing);
        if(split > 1)
        {
            const double ws = (double)split * v.P * v.Q * class_acc_bytes(v.cls);
            // partials out and back, second launch; partials that fit the 256 MiB last-level
            // cache never reach HBM
            const double bw = ws <= 160e6 ? dev.hbm_gbs * 1e3 * 1.0 : dev.hbm_gbs * 1e3 * 0.6;
            // the reduction walks the slices one after another; and short slices are mostly prologue
            // (512^3 in 8 slices against 4: f32 14.0 / 11.9 us, complex f32 24.5 / 20.5, 256^3 complex f64 13.5 / 11.3)
            us += 2.0 * ws / bw + 3.0 + 0.25 * split;
        }
        return us;
    }

    std::vector<Choice> rank_choices(const std::vector<const Solution*>& candidates,
                                     const GemmView&                     v,
                                     uint64_t                            max_ws,
                                     const DeviceModel&                  dev)
    {
        std::vector<Choice> out;
        for(const Solution* s : candidates)
        {
            if(!s || !solution_fits(*s, v))
                continue;
            const int ktiles = (int)((v.K + s->bk - 1) / s->bk);
            for(int split = 1; split <= 64 && split <= ktiles; split *= 2)
            {
                const uint64_t ws = split > 1 ? (uint64_t)split * (uint64_t)v.P * (uint64_t)v.Q
                                                    * (uint64_t)class_acc_bytes(v.cls)
                                              : 0;
                if(ws > max_ws)
                    break;
                Choice c;
                c.sol      = s;
                c.split_k  = split;
                c.ws_bytes = ws;
                c.est_us   = estimate_us(*s, v, split, dev);
                out.push_back(c);
            }
        }
        std::stable_sort(out.begin(), out.end(), [](const Choice& a, const Choice& b) { return a.est_us < b.est_us; });
        return out;
    }
}
