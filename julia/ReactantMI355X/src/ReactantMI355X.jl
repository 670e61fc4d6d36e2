# ReactantMI355X: routes Reactant.jl's non-sharded PJRT path to libreactant_mi355x.so.
#
# UNTESTED: no Julia in the container this was written in.  Written against the reference
# sources cited at each definition; the Python mirror (reactant.jl_amd/__init__.py) drives the
# same C entry points and is what the test suite runs.
#
#     using Reactant, ReactantMI355X
#     Reactant.set_default_backend("gpu")          # resolves to the "rocm" backend registered here
#     x = Reactant.to_rarray(rand(Float32, 1024));  f = @compile sum(sin.(x))
#
# How it hooks in.  Reactant's PJRT wrappers (src/xla/PJRT/{Client,Device,Buffer,Future,
# LoadedExecutable}.jl) are `Ptr{Cvoid}` holders whose methods call the generated bindings
# `Reactant.MLIR.API.<Name>` (src/mlir/libMLIR_h.jl), each a `@ccall mlir_c.<Name>(...)` into
# libReactantExtra.  This package redefines those bindings (routing.jl): a call whose handle was
# created by libreactant_mi355x.so (`RxOwns`) goes to that library, every other call goes to
# libReactantExtra as before, so CPU clients, tracing and the MLIR passes are untouched and a
# ConcretePJRTArray keeps its field types.  A client of this library is made by a backend
# registered under the platform name "rocm" (client.jl); compilation hands the module over as
# text (compile.jl); execution goes through the routed `XLAExecuteSharded` binding (execute.jl).
#
# Redefining methods of another package cannot be precompiled.
__precompile__(false)

module ReactantMI355X

using Libdl: Libdl
using Reactant: Reactant
const XLA = Reactant.XLA
const PJRT = Reactant.XLA.PJRT
const API = Reactant.MLIR.API

const LIB = Ref{Ptr{Cvoid}}(C_NULL)
const SYMS = Dict{Symbol,Ptr{Cvoid}}()

"Address of an exported function of libreactant_mi355x.so (include/reactant_mi355x.h)."
function sym(name::Symbol)
    p = get(SYMS, name, C_NULL)
    if p == C_NULL
        LIB[] == C_NULL && error("ReactantMI355X: libreactant_mi355x.so is not loaded")
        p = Libdl.dlsym(LIB[], name)
        SYMS[name] = p
    end
    return p
end

"Was this client / device / buffer / executable / future handle created by libreactant_mi355x.so?"
@inline function owns(p::Ptr)
    (p == C_NULL || LIB[] == C_NULL) && return false
    return ccall(sym(:RxOwns), Cint, (Ptr{Cvoid},), p) != 0
end
@inline owns(x) = false

# the callback behind the library's `ReactantThrowError` pointer (same behaviour as XLA.reactant_err, src/xla/Utils.jl:13-15)
function throw_reactant_error(msg::Cstring)::Cvoid
    throw(XLA.ReactantInternalError(Base.unsafe_string(msg)))
end

function library_path()
    haskey(ENV, "REACTANT_MI355X_LIB") && return ENV["REACTANT_MI355X_LIB"]
    here = joinpath(@__DIR__, "..", "..", "..", "reactant.jl_amd", "libreactant_mi355x.so")
    return isfile(here) ? abspath(here) : "libreactant_mi355x.so"
end

include("routing.jl")
include("client.jl")
include("compile.jl")
include("execute.jl")

function __init__()
    # RTLD_LOCAL: libReactantExtra exports the same names and stays the default for every handle it owns
    LIB[] = Libdl.dlopen(library_path(), Libdl.RTLD_NOW | Libdl.RTLD_LOCAL)
    # errors raised inside the library become Julia exceptions, as for libReactantExtra
    # (src/xla/XLA.jl:203-204, src/xla/Utils.jl:13-15)
    errptr = convert(Ptr{Ptr{Cvoid}}, Libdl.dlsym(LIB[], :ReactantThrowError))
    unsafe_store!(errptr, @cfunction(throw_reactant_error, Cvoid, (Cstring,)))
    ccall(sym(:InitializeLogs), Cvoid, ())
    install_routes!()
    install_compile!()
    install_execute!()
    install_cost_analysis!()
    register!()
    return nothing
end

end # module
