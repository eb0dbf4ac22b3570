// Dense univariate polynomial over Fr, host side: the interface of the reference's
// include/polynomial.cuh:8-44 / src/polynomial.cu.
#pragma once
#include <iosfwd>
#include <vector>
#include "fr.hpp"

class Polynomial {
public:
    Polynomial();
    Polynomial(int degree);
    Polynomial(int degree, Fr* coefficients);
    Polynomial(const Polynomial& other) = default;
    Polynomial(const Fr& constant);
    Polynomial(const std::vector<Fr>& coefficients);   // low to high

    Polynomial& operator=(const Polynomial& other) = default;

    Polynomial operator+(const Polynomial& other) const;
    Polynomial operator-(const Polynomial& other) const;
    Polynomial operator*(const Polynomial& other) const;
    Polynomial operator*(const Fr& val) const;
    Polynomial operator-() const;

    Polynomial& operator+=(const Polynomial& other);
    Polynomial& operator-=(const Polynomial& other);
    Polynomial& operator*=(const Polynomial& other);

    Fr operator()(const Fr& x) const;     // Horner
    Fr operator()(const int& x) const;    // only meaningful for x = 0 and x = 1, as in the reference

    int getDegree() const { return (int)c_.size() - 1; }
    void setCoefficients(int degree, Fr* coefficients);
    const std::vector<Fr>& coefficients() const { return c_; }

    static Polynomial eq(const Fr& u);              // (1-u) + (2u-1) t
    static Fr eq(const Fr& u, const Fr& v);         // 2uv - u - v + 1

    friend std::ostream& operator<<(std::ostream& os, const Polynomial& poly);

private:
    std::vector<Fr> c_;
};
