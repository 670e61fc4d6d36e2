# Execution.
#
# Reference: `XLA.execute_sharded(exec::PJRT.LoadedExecutable, device::PJRT.Device, inputs, donated,
# Val(n_outs))` (src/xla/PJRT/LoadedExecutable.jl:175-246) is a generated function with two bodies:
# outside precompilation it emits LLVM IR that calls the symbol `XLAExecuteSharded`, which
# XLA.__init__ binds to libReactantExtra's address in Julia's JIT (src/xla/XLA.jl:244-258); while
# precompiling it calls the binding `MLIR.API.XLAExecuteSharded` with `Ref`s.  The JIT symbol
# cannot be rebound after the fact, so this package replaces the method with one that always takes
# the second form; the binding is routed by the owner of `exec` (routing.jl).  The cost against the
# llvmcall form is four small `Ref` allocations per call.
#
# Protocol kept by the library (deps/ReactantExtra/API.cpp:1585-1630): one owning buffer handle per
# result, `futures[] = 1` and one future per result; a donated argument gives up its storage.

function install_execute!()
    Core.eval(
        PJRT,
        quote
            function XLA.execute_sharded(
                exec::LoadedExecutable,
                device::Device,
                inputs::NTuple{N,Ptr{Cvoid}},
                donated_args::NTuple{N,UInt8},
                ::Val{n_outs},
            ) where {N,n_outs}
                args = Ref(inputs)
                donate = Ref(donated_args)
                outputs = Ref{NTuple{n_outs,Ptr{Cvoid}}}()
                future_res = Ref{NTuple{n_outs,Ptr{Cvoid}}}()
                has_futures = Ref{UInt8}(0)
                GC.@preserve exec device args donate outputs future_res has_futures begin
                    MLIR.API.XLAExecuteSharded(
                        exec.exec,
                        Cint(N),
                        Base.unsafe_convert(Ptr{Ptr{Cvoid}}, Base.unsafe_convert(Ptr{Cvoid}, args)),
                        device.device,
                        Base.unsafe_convert(Ptr{UInt8}, Base.unsafe_convert(Ptr{Cvoid}, donate)),
                        Cint(n_outs),
                        Base.unsafe_convert(Ptr{Ptr{Cvoid}}, Base.unsafe_convert(Ptr{Cvoid}, outputs)),
                        Base.unsafe_convert(Ptr{UInt8}, has_futures),
                        Base.unsafe_convert(Ptr{Ptr{Cvoid}}, Base.unsafe_convert(Ptr{Cvoid}, future_res)),
                    )
                end
                outs, futs, with_futures = outputs[], future_res[], has_futures[] != 0
                return ntuple(Val(n_outs)) do i
                    Base.@_inline_meta
                    (AsyncBuffer(Buffer(outs[i]), with_futures ? Future(futs[i]) : nothing),)
                end
            end
        end,
    )
    return nothing
end

"""
    execute_no_alloc!(exec, args, results)

Run `exec` with caller-owned result buffers (made ahead of time with `similar` / `UninitPJRTBuffer`
of the result types); the plan's temporaries live in a static 4 MiB device array, so nothing is
allocated.  No counterpart in the reference.  Plans with larger temporaries are refused.
"""
function execute_no_alloc!(exec::PJRT.LoadedExecutable, args::Vector{PJRT.Buffer}, results::Vector{PJRT.Buffer})
    owns(exec.exec) || error("execute_no_alloc!: not an executable of libreactant_mi355x.so")
    a = Ptr{Cvoid}[b.buffer for b in args]
    r = Ptr{Cvoid}[b.buffer for b in results]
    GC.@preserve exec args results a r begin
        rc = ccall(
            sym(:RxExecuteNoAlloc), Cint, (Ptr{Cvoid}, Cint, Ptr{Ptr{Cvoid}}, Cint, Ptr{Ptr{Cvoid}}),
            exec.exec, length(a), a, length(r), r,
        )
    end
    rc == 0 || error("RxExecuteNoAlloc failed: " * unsafe_string(ccall(sym(:RxLastError), Cstring, ())))
    return results
end

"""
    XLA.cost_analysis(exec::PJRT.LoadedExecutable)

Reference: `cost_analysis(exec)` asks every HLO module of the executable
(src/xla/LoadedExecutable.jl:14-18 -> `pjrt_hlo_module_cost_analysis_properties`, src/xla/PJRT/Client.jl:83-90).
An executable of this library keeps no HLO module (`get_hlo_modules` returns none), so the same
`JLHloCostAnalysisProperties` comes from `RxExecutableCostAnalysis`, counted over the StableHLO module
the executable was compiled from.
"""
function install_cost_analysis!()
    Core.eval(
        PJRT,
        quote
            function XLA.cost_analysis(exec::LoadedExecutable)
                $(owns)(exec.exec) || return invoke(XLA.cost_analysis, Tuple{XLA.AbstractLoadedExecutable}, exec)
                props = Ref{MLIR.API.JLHloCostAnalysisProperties}()
                GC.@preserve exec props begin
                    ccall($(sym)(:RxExecutableCostAnalysis), Cvoid, (Ptr{Cvoid}, Ptr{Cvoid}), exec.exec, props)
                end
                return props[]
            end
        end,
    )
    return nothing
end
